// The small-tile fused apply of decode.hip (one workgroup per (<= 16 tokens of one slot, column
// range), both products on the matrix cores; same arithmetic, same order, same bits) with the grid
// laid over the SLOTS instead of over the tiles.  Computes what the reference computes with a
// shrink launch, a temporary [slices, T, r] tensor and one or two expand launches
// (nanovllm_voxcpm/lora.py:291-381, lora_ops/triton_ops/lora_shrink_op.py:16-173,
// lora_expand_op.py:11-91).
//
// Why a second grid.  A decode launch lives for three to five trips to memory, and in the
// tile-major kernel the first of them fetches nothing but the 128-byte tile record: which slot a
// workgroup serves is written there, so not one operand can be requested before it has arrived.
// More than half of a decode launch's bytes are A[slot] and B[slot], and their addresses need the
// slot id only.  Here the slot id IS the workgroup index: workgroup (x, range, z) serves slot
// 8 z + x, so it requests the slot's record (its first sixteen tokens) and right behind it, without
// waiting, every A line it will need; the record is waited for while they are on their way, and
// only the x and y rows (whose addresses are token indices) hang on it.  The B rows, which need the
// slot id alone as well, go out behind the x rows: nothing uses them before the expand, and a
// compute unit hands over only so many requests at a time, so in front of the record's wait they
// held the x rows up (gate_up: 32 KB of A and 32 KB of B per workgroup).  For that
// to be true the weight pointers must not need a fetch either: they are leading kernel arguments,
// which arrive preloaded in scalar registers with the wavefront (14 dwords: the record list, two
// slices' A and B, their widths, and a packed word).  A slot without tokens costs its workgroups
// the A lines they requested in vain; they leave as soon as the record says so.
//
// Tiles behind a slot's first sixteen tokens are taken by further workgroups of the same launch
// (z beyond the slot layers), which learn their slot from their record like the tile-major
// kernel: a batch with every token on one adapter spreads over as many workgroups as before.
//
// Long K (KP > 1).  What a compute unit can take in per unit of time is what bounds a decode
// launch (about 35 bytes per cycle, whether the lines come from HBM or from the L2), and with one
// workgroup per column range every range pulls ALL of x's tile and of A[slot]: at K = 4096 that is
// 256 KB per workgroup against 16 KB of B and y.  With KP > 1 the KP workgroups of a tile each take
// one K part AND one column range: a workgroup multiplies its part, publishes the 16 x r partial
// sums as tagged 64-bit words in the workspace's exchange area, picks up the other parts'
// words, adds all parts in part order (so every workgroup of the tile holds the same bits) and
// expands its columns.  The hand-over follows the protocol of split.hip: words are valid when
// their tag is the workspace's generation + 1, every workgroup of the grid counts itself once,
// the last one advances the generation, nothing is ever cleared.  Waiting is bounded: a workgroup
// whose partners' words are not there in time multiplies their parts itself, in their order.
#include "common.h"
#include "launch.h"

namespace mlora {

namespace {

constexpr int kNW = 8;  // wavefronts per workgroup

MLORA_TRACE_DECL

// What a workgroup needs to know of its column range.
struct Range {
  const void* a;
  const void* b;
  int n, y_col, n0, n1;
};

// One tile.  EARLY: the slot is known from the workgroup index (slot_early) and A[slot] is
// requested before the record has arrived; otherwise the record names the slot.
// The operand path is the staged one of decode.hip: x rows and A rows of a wavefront's K range are
// fetched row-contiguously (sixteen lanes per 256 bytes of a row), turned into MFMA operand layout
// through a private LDS block per wavefront, and the expand runs with the tokens as MFMA rows.
// What the workgroups of a tile need to hand each other partial sums (KP > 1).
struct Exchange {
  uint32_t* ws;    // workspace head
  int spin_ticks;  // bound of the wait for the partners' words, in ticks of the 100 MHz clock (< 0: never accept any)
  int trusted;     // the head is known to be in a launch's or the initial state without carrying the signature
};

typedef unsigned long long u64;

// GR (with MASKED): the buffers' rank is `rbuf` < R, a multiple of eight: rows of A[slot] are rbuf * K
// apart and B rows rbuf elements long; whatever lies beyond rbuf is treated like the ranks beyond
// an adapter's own (requests clamped into the buffers, values masked).
template <typename T, int R, int KSPW, int KP, bool MASKED, bool GR, int SA, bool EARLY>
__device__ __forceinline__ void slot_tile(const int32_t* __restrict__ rec, const int slot_early, const int early_ok, const int rbuf_arg, const Range sp,
                                          const int y_col0, const int y_col1, const int y_col2, const int slice, const void* __restrict__ xv,
                                          void* __restrict__ yv_, const int64_t xs, const int64_t ys,
                                          const int num_slots, const float scaling, const int32_t* __restrict__ eff_rank,
                                          const uint32_t check, int32_t* __restrict__ plan_hdr, const Exchange xc, float* __restrict__ s_red,
                                          T* __restrict__ s_hi, T* __restrict__ s_lo, i32x4* __restrict__ s_stage, int* __restrict__ s_ok) {
  constexpr int RB = (R + 15) / 16;      // 16-rank blocks of the shrink output
  constexpr int KSTEPS = (R + 31) / 32;  // MFMA k-steps of the expand
  constexpr int HSTRIDE = R + 8;         // padded LDS row of the intermediate
  constexpr int NT = kNW * kWave;
  constexpr int ROUNDS = KSPW / 4;       // groups of four k-steps per wavefront
  constexpr int KPART = 32 * kNW * KSPW;  // columns of x and A one workgroup multiplies
  constexpr int K = KPART * KP;           // row length of A[slot]
  constexpr int WORDS = RB * 256;         // partial sums of one (tile, K part), in the order of the shared sum below
  constexpr int EPT = (WORDS + NT - 1) / NT;  // of which a thread holds this many
  constexpr int kStageRow = 17;          // 16 chunks of 16 bytes + one of padding
  constexpr int SB = RB < 2 ? RB : 2;    // 16-rank blocks of A staged together
  constexpr bool K16 = R == 16;          // expand on the 16x16x16 MFMA: 64-bit operand pieces
  static_assert(!GR || (MASKED && R >= 32), "buffers of a rank between the instances' take the masked code of the next instance up");
  static_assert(KSPW >= 4 && KSPW % 4 == 0, "the k-steps of a wavefront are taken four at a time");

  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int lr = lane & 15, lg = lane >> 4;
  const int rbuf = GR ? rbuf_arg : R;  // rank of the buffers: row count of A[slot], row length of B

  // ---- requests that depend on nothing but the workgroup index --------------------------------
  // (the token rows as a vector load, four per lane group: all sixteen through the scalar cache
  // into scalar registers measured slower, 556 -> 598 us per decode step in the tile-major kernel)
  const i32x4 rows4 = *reinterpret_cast<const i32x4*>(rec + MLORA_SMALL_TILE_ROWS + 4 * lg);  // tokens 4*lg .. 4*lg+3
  const i32x4 rec0 = *reinterpret_cast<const i32x4*>(rec);                                     // slot, count, start, check
  int eff_early = R;
  if constexpr (MASKED && EARLY) {
    if (eff_rank) eff_early = eff_rank[slot_early];
  }
  const RankPrefetch ranks = rank_prefetch((MASKED && !EARLY) ? eff_rank : nullptr, num_slots, lane);
  if constexpr (EARLY) __builtin_amdgcn_sched_barrier(0);  // the record's requests go out first

  const int kp = KP > 1 ? static_cast<int>(blockIdx.y) : 0;  // this workgroup's K part (and column range)
  const int ks0 = kp * (KPART / 32) + wave * KSPW;
  // the workspace's {generation, arrivals, check word} and signature (KP > 1): requested with the record
  uint32_t* const tstate = KP > 1 ? xc.ws + kWsTileOff / 4 : nullptr;
  uint32_t signature = 0, generation = 0, arrivals0 = 0, gen_check = 0;
  if constexpr (KP > 1) {
    signature = xc.ws[0];
    generation = tstate[0];
    arrivals0 = tstate[1];
    gen_check = tstate[2];
  }
  i32x4 ast[RB][4 * ROUNDS];
  Pack8 bop[SA][4][KSTEPS];
  // every A line of this wavefront's K range
  auto request_a = [&](const int slot, const int rb_n) {
    const T* A = static_cast<const T*>(sp.a) + static_cast<int64_t>(slot) * rbuf * K;
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) {
      const int64_t koff = static_cast<int64_t>(ks0 + 4 * r) * 32 + (lane & 15) * 8;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
          const int rr = rb * 16 + 4 * lg + i;
          if (!MASKED || EARLY || RB == 1 || rb < rb_n) ast[rb][4 * r + i] = load128(A + static_cast<int64_t>(rr < rbuf ? rr : rbuf - 1) * K + koff);
          else ast[rb][4 * r + i] = i32x4{0, 0, 0, 0};
        }
      }
    }
  };
  // the B rows of its spans
  auto request_b = [&](const int slot) {
    const T* B = static_cast<const T*>(sp.b) + static_cast<int64_t>(slot) * sp.n * rbuf;
#pragma unroll
    for (int s = 0; s < SA; ++s) {
      const int c0 = sp.n0 + (wave + s * kNW) * 64;
      // requested whether the span exists or not (addresses clamped into the range)
      if constexpr (K16) {
        // a span's 64 B rows of 32 bytes are 2 KB of contiguous memory: fetched as such
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          int n = c0 + 32 * h + (lane >> 1);
          n = n < sp.n1 ? n : sp.n1 - 1;
          bop[s][h][0].raw = load128(B + static_cast<int64_t>(n) * R + (lane & 1) * 8);
        }
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          int n = c0 + 4 * lr + j;
          n = n < sp.n1 ? n : sp.n1 - 1;
#pragma unroll
          for (int ks = 0; ks < KSTEPS; ++ks) {
            int kc = (lg + 4 * ks) & (R / 8 - 1);
            if (GR && kc * 8 >= rbuf) kc = rbuf / 8 - 1;  // (masked where it is used)
            bop[s][j][ks].raw = load128(B + static_cast<int64_t>(n) * rbuf + kc * 8);
          }
        }
      }
    }
  };
  // The requests made in vain by a workgroup that turns out to have no work: waited for, and named
  // as used on that path too, so that the compiler cannot move them behind the test on the record
  // (left to itself it sinks every load into the only path that uses it).
  auto settle_requests = [&]() {
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int j = 0; j < 4 * ROUNDS; ++j) asm volatile("" ::"v"(ast[rb][j]));
  };
  if constexpr (EARLY) request_a(slot_early, RB);
  // (everything above is requested before anything below is scheduled)
  __builtin_amdgcn_sched_barrier(0);

  // ---- the record is here (the weights, when requested early, are still on their way) ---------
  const int slot = EARLY ? slot_early : rec0[0];
  const int m = rec0[1];
  const int matches = int(static_cast<uint32_t>(rec0[3]) == check);
  // (every word of the record takes part in the test: a word that nothing reads is a register the
  // compiler hands out again while the request is still on its way, and the write to it then
  // waits for the record in the middle of the requests for the weights)
  const int usable = matches & early_ok & int(m > 0) & int(slot >= 0) & int(slot < num_slots) & int(sp.n0 < sp.n1) &
                     int(__builtin_amdgcn_readfirstlane(rows4[0]) >= 0) & int(rec0[2] >= 0) & int(!EARLY || rec0[0] == slot_early);
  // KP > 1: the exchange area can be used when the head is in the state a launch (or the
  // initialisation) left it in.  Every workgroup of the grid, with or without work, reports once
  // that it reads the area no more; the last one advances the generation.
  const uint32_t tag = generation + 1u;
  const bool xok = KP > 1 && (xc.trusted | ws_state_ok(signature, generation, arrivals0, gen_check, gridDim.x * gridDim.y * gridDim.z));
  // The count comes back from the memory system long after it was sent: a working workgroup sends
  // it behind its last barrier (count_sent, by the last wavefront, which has the fewest spans to
  // expand) and looks at what came back when its stores are out (count_seen).
  const bool counter = KP > 1 && xok && tid == NT - kWave;
  uint32_t arrivals_before = 0;
  auto count_sent = [&]() {
    if constexpr (KP > 1) {
      if (counter) arrivals_before = __hip_atomic_fetch_add(tstate + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  };
  auto count_seen = [&]() {
    if constexpr (KP > 1) {
      if (counter && arrivals_before + 1u == gridDim.x * gridDim.y * gridDim.z) {
        const uint32_t next = tag == 0xffffffffu ? 0u : tag;  // so that generation + 1, the next tag, is never 0
        __hip_atomic_store(tstate + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(tstate + 2, next ^ kWsGenCheck, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(tstate, next, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  };
  auto count_done = [&]() {
    count_sent();
    count_seen();
  };
  if (!usable) {
    count_done();
    // a plan that was built for another batch shape (or never built): count the launch that found
    // it so, once (the first workgroup's record exists in every plan)
    if (!matches && EARLY && blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0 && tid == 0 && plan_hdr)
      atomicAdd(plan_hdr + MLORA_PLAN_REJECTED, 1);
    if constexpr (EARLY) settle_requests();
    return;
  }
  MLORA_STAMP(1);
  // (the column offset of the slice inside y comes with the arguments that are not preloaded:
  // selected here, behind the wait for the record, it holds nothing up)
  const int y_col = slice == 0 ? y_col0 : slice == 1 ? y_col1 : y_col2;

  int eff = R;
  if constexpr (MASKED) {
    if constexpr (EARLY) {
      const int e = __builtin_amdgcn_readfirstlane(eff_early);
      eff = e < 0 ? 0 : e > R ? R : e;
    } else {
      eff = rank_pick(ranks, eff_rank, num_slots, slot, R);
    }
    if (GR && eff > rbuf) eff = rbuf;
    if (eff == 0) {
      count_done();
      if constexpr (EARLY) settle_requests();
      return;
    }
  }
  const int rb_n = MASKED ? (eff + 15) >> 4 : RB;  // 16-rank blocks of A in use
  if constexpr (!EARLY) request_a(slot, rb_n);

  // ---- the rows the record names --------------------------------------------------------------
  i32x4 xst[4 * ROUNDS];
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) {
    const int64_t koff = static_cast<int64_t>(ks0 + 4 * r) * 32 + (lane & 15) * 8;
#pragma unroll
    for (int i = 0; i < 4; ++i) xst[4 * r + i] = load128(static_cast<const T*>(xv) + static_cast<int64_t>(rows4[i]) * xs + koff);
  }
  // (the B rows behind the x rows: they are not needed before the expand, and in front of the
  // record's wait they would hold the x rows up for as long as it takes to hand them over)
  request_b(slot);
  uint2 yq[SA][4];  // four columns of four tokens per lane and span
  T* const ycols = static_cast<T*>(yv_) + y_col;
  auto request_y = [&](int c0, uint2(&yy)[4]) {
    const int c = c0 + 4 * lr < sp.n1 ? c0 + 4 * lr : sp.n1 - 4;
#pragma unroll
    for (int i = 0; i < 4; ++i) yy[i] = *reinterpret_cast<const uint2*>(ycols + static_cast<int64_t>(rows4[i]) * ys + c);
  };
#pragma unroll
  for (int s = 0; s < SA; ++s) request_y(sp.n0 + (wave + s * kNW) * 64, yq[s]);
  MLORA_STAMP(2);  // every load is issued

  // ---- shrink: H[token, rank] partial over this wavefront's K range ----------------------------
  i32x4* stage = s_stage + wave * (1 + SB) * 16 * kStageRow;
  // x rows and A rows, fetched row-contiguously, through the wavefront's LDS block into operand
  // layout, and multiplied: k-steps in ascending order
  auto stage_and_multiply = [&](const i32x4(&xs_)[4 * ROUNDS], const i32x4(&as_)[RB][4 * ROUNDS], f32x4(&acc)[RB], const bool clear_blocks) {
    Pack8 xa[4], aw[RB][4];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) acc[rb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) {
#pragma unroll
      for (int i = 0; i < 4; ++i) stage[(4 * lg + i) * kStageRow + (lane & 15)] = xs_[4 * r + i];
#pragma unroll
      for (int p = 0; p < RB / SB; ++p) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
#pragma unroll
          for (int sb = 0; sb < SB; ++sb) {
            i32x4 v = as_[p * SB + sb][4 * r + i];
            // rank blocks the adapter does not have were requested before its rank was known: they
            // never reach a multiplier
            if (MASKED && RB > 1 && clear_blocks && p * SB + sb >= rb_n) v = i32x4{0, 0, 0, 0};
            stage[((1 + sb) * 16 + 4 * lg + i) * kStageRow + (lane & 15)] = v;
          }
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (p == 0) xa[i].raw = stage[lr * kStageRow + 4 * i + lg];
#pragma unroll
          for (int sb = 0; sb < SB; ++sb) aw[p * SB + sb][i].raw = stage[((1 + sb) * 16 + lr) * kStageRow + 4 * i + lg];
        }
        __builtin_amdgcn_wave_barrier();  // the block is rewritten by the next pass or round (and later by the expand)
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) acc[rb] = Mma<T>::run(xa[i], aw[rb][i], acc[rb]);
      }
    }
  };
  // Sum of the wavefronts' partial tiles, wavefront 0 first: out[j] is word tid + j * NT.
  // D layout: lane holds H[token 4*(lane/16)+i][rank lane%16].
  auto sum_wavefronts = [&](const f32x4(&acc)[RB], float(&out)[EPT]) {
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) *reinterpret_cast<f32x4*>(&s_red[((wave * RB + rb) * 64 + lane) * 4]) = acc[rb];
    MLORA_STAMP(3);
    __syncthreads();
    MLORA_STAMP(4);
#pragma unroll
    for (int j = 0; j < EPT; ++j) {
      const int e = tid + j * NT;
      float sum = 0.f;
      if (WORDS % NT == 0 || e < WORDS) {
        const int rb = e >> 8, ln = (e & 255) >> 2, i = e & 3;
#pragma unroll
        for (int w = 0; w < kNW; ++w) sum += s_red[((w * RB + rb) * 64 + ln) * 4 + i];
      }
      out[j] = sum;
    }
  };
  f32x4 acc[RB];
  float total[EPT];
  if (KP > 1 && tid == 0) *s_ok = 1;  // (seen by everyone behind the barrier of the sum below)
  stage_and_multiply(xst, ast, acc, EARLY);
  sum_wavefronts(acc, total);

  if constexpr (KP > 1) {
    // ---- the other K parts: from the tile's other workgroups, or multiplied here -----------------
    u64* const xchg = reinterpret_cast<u64*>(reinterpret_cast<char*>(xc.ws) + kWsXchgOff) +
                      static_cast<int64_t>(blockIdx.z * 8 + blockIdx.x) * (KP * WORDS);  // the KP parts of this tile
    float part[KP][EPT];
#pragma unroll
    for (int q = 0; q < KP; ++q)
#pragma unroll
      for (int j = 0; j < EPT; ++j) part[q][j] = 0.f;
    if (xok) {
#pragma unroll
      for (int j = 0; j < EPT; ++j) {
        const int e = tid + j * NT;
        if (WORDS % NT == 0 || e < WORDS)
          __hip_atomic_store(xchg + kp * WORDS + e, (static_cast<u64>(tag) << 32) | __float_as_uint(total[j]), __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_WORKGROUP);
      }
    }
    MLORA_STAMP(9);  // this workgroup's partial sums are on their way to the L2
    int ok = xok && xc.spin_ticks >= 0;
    if (ok) {
      const long long t0 = wall_clock64();
      for (;;) {
        // every part's words are requested together, this workgroup's own among them (a request
        // behind a test on the part number is a round trip of its own); its own are not looked at
        u64 w[KP][EPT];
#pragma unroll
        for (int q = 0; q < KP; ++q) {
#pragma unroll
          for (int j = 0; j < EPT; ++j) {
            const int e = (WORDS % NT == 0 || tid + j * NT < WORDS) ? tid + j * NT : 0;
            w[q][j] = __hip_atomic_load(xchg + q * WORDS + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
        }
        bool all = true;
#pragma unroll
        for (int q = 0; q < KP; ++q) {
#pragma unroll
          for (int j = 0; j < EPT; ++j) {
            const bool mine = !(WORDS % NT == 0 || tid + j * NT < WORDS) || q == kp;
            all &= mine | (static_cast<uint32_t>(w[q][j] >> 32) == tag);
            part[q][j] = __uint_as_float(static_cast<uint32_t>(w[q][j]));
          }
        }
        if (__builtin_amdgcn_ballot_w64(all) == __builtin_amdgcn_ballot_w64(true)) break;
        if (wall_clock64() - t0 >= xc.spin_ticks) { ok = 0; break; }
        __builtin_amdgcn_s_sleep(1);
      }
      if (!ok && xc.spin_ticks > 0 && lane == 0) atomicAdd(xc.ws + kWsTimeoutsWord, 1u);  // diagnostic: a wait ran out
    }
    MLORA_STAMP(10);  // the wait for the partners is over
    // one verdict for the workgroup (through a flag in LDS: the library's block-wide AND reads the
    // launch's shape from memory first, two trips); the barrier also ends the reading of s_red
    if (!ok) *s_ok = 0;
    __syncthreads();
    ok = *s_ok;
    if (!ok) {
      // every other part multiplied here as its own workgroup multiplies it
      for (int q = 0; q < KP; ++q) {
        if (q == kp) continue;
        i32x4 xo[4 * ROUNDS], ao[RB][4 * ROUNDS];
        const T* A = static_cast<const T*>(sp.a) + static_cast<int64_t>(slot) * rbuf * K;
#pragma unroll
        for (int r = 0; r < ROUNDS; ++r) {
          const int64_t koff = static_cast<int64_t>(q * (KPART / 32) + wave * KSPW + 4 * r) * 32 + (lane & 15) * 8;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            xo[4 * r + i] = load128(static_cast<const T*>(xv) + static_cast<int64_t>(rows4[i]) * xs + koff);
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
              const int rr = rb * 16 + 4 * lg + i;
              if (!MASKED || RB == 1 || rb < rb_n) ao[rb][4 * r + i] = load128(A + static_cast<int64_t>(rr < rbuf ? rr : rbuf - 1) * K + koff);
              else ao[rb][4 * r + i] = i32x4{0, 0, 0, 0};
            }
          }
        }
        f32x4 acc2[RB];
        float got[EPT];
        stage_and_multiply(xo, ao, acc2, false);
        sum_wavefronts(acc2, got);
        __syncthreads();  // s_red is rewritten by the next part
#pragma unroll
        for (int qq = 0; qq < KP; ++qq) {
          if (qq == q) {
#pragma unroll
            for (int j = 0; j < EPT; ++j) part[qq][j] = got[j];
          }
        }
      }
    }
    // all parts added up in part order, this workgroup's own at its place
#pragma unroll
    for (int j = 0; j < EPT; ++j) {
      const float own = total[j];
      float sum = 0.f;
#pragma unroll
      for (int q = 0; q < KP; ++q) sum += q == kp ? own : part[q][j];
      total[j] = sum;
    }
  }
#pragma unroll
  for (int j = 0; j < EPT; ++j) {
    const int e = tid + j * NT;
    if (WORDS % NT == 0 || e < WORDS) {
      const int rb = e >> 8, ln = (e & 255) >> 2, i = e & 3;
      const int tok = 4 * (ln >> 4) + i, r = rb * 16 + (ln & 15);
      if (r < R) {
        const float v = (!MASKED || r < eff) ? total[j] * scaling : 0.f;  // ranks the adapter does not have contribute nothing
        const T hi = from_f32<T>(v);
        s_hi[tok * HSTRIDE + r] = hi;
        s_lo[tok * HSTRIDE + r] = from_f32<T>(v - to_f32(hi));
      }
    }
  }
  __syncthreads();
  MLORA_STAMP(5);  // the intermediate is in LDS
  // This workgroup reads the exchange area no more.  Sent behind the last barrier: the compiler
  // waits for the count on the spot (it is requested inside a branch), and in front of a barrier
  // the whole workgroup would wait with the wavefront that sent it.
  count_sent();

  // ---- expand: tokens as MFMA rows, lane holds out[token 4 * lg + i][column c0 + 4 * lr + j] ----
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
  auto finish_span = [&](int c0, Pack8(&bo)[4][KSTEPS], uint2(&yy)[4]) {
    f32x4 out[4];
    uint2 pieces[4];
    if constexpr (K16) {
      if (MASKED && eff < R) {
        mask_ranks(bo[0][0], (lane & 1) * 8, eff);
        mask_ranks(bo[1][0], (lane & 1) * 8, eff);
      }
      // B rows -> operand pieces through the wavefront's LDS block: four rows (128 bytes) per
      // group, groups 144 bytes apart.  MFMA j of lane (lr, lg) takes ranks 4*lg .. 4*lg+3 of
      // column c0 + 4*lr + j.
      char* blk = reinterpret_cast<char*>(stage);
      *reinterpret_cast<i32x4*>(blk + (lane >> 3) * 144 + (lane & 7) * 16) = bo[0][0].raw;
      *reinterpret_cast<i32x4*>(blk + ((lane >> 3) + 8) * 144 + (lane & 7) * 16) = bo[1][0].raw;
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int j = 0; j < 4; ++j) pieces[j] = *reinterpret_cast<const uint2*>(blk + lr * 144 + j * 32 + lg * 8);
      __builtin_amdgcn_wave_barrier();
    } else if (MASKED && eff < R) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) mask_ranks(bo[j][ks], ((lg + 4 * ks) & (R / 8 - 1)) * 8, eff);
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
          out[j] = Mma<T>::run(hlo[ks], bo[j][ks], out[j]);
          out[j] = Mma<T>::run(hop[ks], bo[j][ks], out[j]);
        }
      }
    }
    const int c = c0 + 4 * lr;
    // (the y values are taken as they are only here: unpacked where they were requested, the
    // wavefront would wait for their arrival before the shrink)
#pragma unroll
    for (int i = 0; i < 4; ++i) asm volatile("" : "+v"(yy[i].x), "+v"(yy[i].y));
    if (c < sp.n1) {
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
  for (int s = 0; s < SA; ++s) {
    const int c0 = sp.n0 + (wave + s * kNW) * 64;
    if (c0 < sp.n1) finish_span(c0, bop[s], yq[s]);
  }
  MLORA_STAMP(6);
  count_seen();
#ifdef MLORA_TRACE
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  MLORA_STAMP(7);
  __syncthreads();
  MLORA_STAMP(8);
#endif
}

// Leading arguments up to `rbuf` (14 dwords) arrive preloaded in scalar registers: everything the
// early requests need.  packed = columns per range / 64 | ranges of slice 0 << 8 | slots << 16.
// A launch of one slice passes n1 = 0 (blockIdx.y never reaches a second slice).
// KP > 1: one slice, blockIdx.y is the workgroup's K part and column range alike (ranges of slice 0 = KP).
template <typename T, int R, int KSPW, int KP, bool MASKED, bool GR, int SA>
__global__ __launch_bounds__(kNW* kWave) void slot_kernel(const int32_t* __restrict__ recs, const void* __restrict__ a0,
                                                          const void* __restrict__ b0, const void* __restrict__ a1,
                                                          const void* __restrict__ b1, int n0, int n1, uint32_t packed, int rbuf,
                                                          const void* __restrict__ xv, void* __restrict__ yv_, int64_t xs, int64_t ys,
                                                          int y_col0, int y_col1, uint32_t check, float scaling,
                                                          const int32_t* __restrict__ eff_rank, int32_t* __restrict__ plan_hdr,
                                                          uint32_t* __restrict__ ws, int spin_ticks, int trusted) {
  constexpr int RB = (R + 15) / 16;
  constexpr int HSTRIDE = R + 8;
  constexpr int kStageRow = 17;
  constexpr int SB = RB < 2 ? RB : 2;
  __shared__ __attribute__((aligned(16))) float s_red[kNW * RB * 64 * 4];
  __shared__ __attribute__((aligned(16))) T s_hi[16 * HSTRIDE];
  __shared__ __attribute__((aligned(16))) T s_lo[16 * HSTRIDE];
  __shared__ __attribute__((aligned(16))) i32x4 s_stage[kNW * (1 + SB) * 16 * kStageRow];
  __shared__ int s_ok;
  MLORA_STAMP(0);

  const int nt = static_cast<int>(packed & 255u) * 64, ranges0 = static_cast<int>((packed >> 8) & 255u);
  const int num_slots = static_cast<int>(packed >> 16);
  const int ri = blockIdx.y;
  const bool second = ri >= ranges0;
  Range sp;
  sp.a = second ? a1 : a0;
  sp.b = second ? b1 : b0;
  sp.n = second ? n1 : n0;
  sp.y_col = 0;  // (selected inside, late)
  sp.n0 = (second ? ri - ranges0 : ri) * nt;
  sp.n1 = sp.n0 + nt < sp.n ? sp.n0 + nt : sp.n;

  // grid (8, column ranges, slot layers + layers of further tiles): blockIdx.x is the XCD, so a
  // slot's column ranges share an L2
  const int zslots = (num_slots + 7) >> 3;
  const Exchange xc{ws, spin_ticks, trusted};
  if (static_cast<int>(blockIdx.z) < zslots) {
    const int s = blockIdx.z * 8 + blockIdx.x;  // its record exists: the list is rounded up to eight
    const int slot = s < num_slots ? s : num_slots - 1;
    slot_tile<T, R, KSPW, KP, MASKED, GR, SA, true>(recs + s * MLORA_SMALL_TILE_WORDS, slot, int(s < num_slots), rbuf, sp, y_col0, y_col1, 0, int(second), xv, yv_,
                                                xs, ys, num_slots, scaling, eff_rank, check, plan_hdr, xc, s_red, s_hi, s_lo, s_stage, &s_ok);
  } else {
    const int q = zslots * 8 + (blockIdx.z - zslots) * 8 + blockIdx.x;
    slot_tile<T, R, KSPW, KP, MASKED, GR, SA, false>(recs + q * MLORA_SMALL_TILE_WORDS, 0, 1, rbuf, sp, y_col0, y_col1, 0, int(second), xv, yv_, xs, ys, num_slots,
                                                 scaling, eff_rank, check, plan_hdr, xc, s_red, s_hi, s_lo, s_stage, &s_ok);
  }
}

// Three slices (the stacked q | k | v projection): six pointers do not fit the fourteen preloaded
// dwords, so the second and third slice's travel as 40-bit offsets from the first one's, in units of
// 16 bytes (+-8 TiB: the slices of a projection are allocations of their own and may lie far apart;
// the launcher takes this kernel only when they fit): their low 32 bits as four arguments, their
// high 8 bits together in a fifth; the widths as 16-bit counts of eight columns.  widths01 = n0 / 8 | n1 / 8 << 16; widths2 = n2 / 8 | ranges of slice 0 << 16 |
// ranges of slices 0 and 1 << 24; packed = columns per range / 64 | slots << 16.
template <typename T, int R, bool MASKED>
__global__ __launch_bounds__(kNW* kWave) void slot_kernel3(const int32_t* __restrict__ recs, const void* __restrict__ a0,
                                                           const void* __restrict__ b0, uint32_t aoff1, uint32_t aoff2, uint32_t boff1, uint32_t boff2,
                                                           uint32_t off_high, uint32_t widths01, uint32_t widths2, uint32_t packed,
                                                           const void* __restrict__ xv, void* __restrict__ yv_, int64_t xs, int64_t ys,
                                                           int y_col0, int y_col1, int y_col2, uint32_t check, float scaling,
                                                           const int32_t* __restrict__ eff_rank, int32_t* __restrict__ plan_hdr) {
  constexpr int RB = (R + 15) / 16;
  constexpr int HSTRIDE = R + 8;
  constexpr int kStageRow = 17;
  constexpr int SB = RB < 2 ? RB : 2;
  __shared__ __attribute__((aligned(16))) float s_red[kNW * RB * 64 * 4];
  __shared__ __attribute__((aligned(16))) T s_hi[16 * HSTRIDE];
  __shared__ __attribute__((aligned(16))) T s_lo[16 * HSTRIDE];
  __shared__ __attribute__((aligned(16))) i32x4 s_stage[kNW * (1 + SB) * 16 * kStageRow];
  __shared__ int s_ok;
  MLORA_STAMP(0);

  const int nt = static_cast<int>(packed & 255u) * 64, num_slots = static_cast<int>(packed >> 16);
  const int cum1 = static_cast<int>((widths2 >> 16) & 255u), cum2 = static_cast<int>(widths2 >> 24);
  const int ri = blockIdx.y;
  const int slice = int(ri >= cum1) + int(ri >= cum2);
  // (offset i: low word off_i, bits 32..39 in byte i of off_high, sign-extended)
  const uint32_t alo = slice == 1 ? aoff1 : aoff2, blo = slice == 1 ? boff1 : boff2;
  const int32_t ahi = static_cast<int8_t>(off_high >> (slice == 1 ? 0 : 8)), bhi = static_cast<int8_t>(off_high >> (slice == 1 ? 16 : 24));
  const int64_t ao = slice == 0 ? 0 : (static_cast<int64_t>(ahi) << 32) | alo, bo = slice == 0 ? 0 : (static_cast<int64_t>(bhi) << 32) | blo;
  Range sp;
  sp.a = static_cast<const char*>(a0) + ao * 16;
  sp.b = static_cast<const char*>(b0) + bo * 16;
  sp.n = 8 * static_cast<int>(slice == 0 ? widths01 & 0xffffu : slice == 1 ? widths01 >> 16 : widths2 & 0xffffu);
  sp.y_col = 0;  // (selected inside, late)
  sp.n0 = (ri - (slice == 0 ? 0 : slice == 1 ? cum1 : cum2)) * nt;
  sp.n1 = sp.n0 + nt < sp.n ? sp.n0 + nt : sp.n;

  const int zslots = (num_slots + 7) >> 3;
  const Exchange xc{nullptr, 0, 0};
  if (static_cast<int>(blockIdx.z) < zslots) {
    const int s = blockIdx.z * 8 + blockIdx.x;
    const int slot = s < num_slots ? s : num_slots - 1;
    slot_tile<T, R, 4, 1, MASKED, false, 1, true>(recs + s * MLORA_SMALL_TILE_WORDS, slot, int(s < num_slots), R, sp, y_col0, y_col1, y_col2, slice, xv,
                                                  yv_, xs, ys, num_slots, scaling, eff_rank, check, plan_hdr, xc, s_red, s_hi, s_lo, s_stage, &s_ok);
  } else {
    const int q = zslots * 8 + (blockIdx.z - zslots) * 8 + blockIdx.x;
    slot_tile<T, R, 4, 1, MASKED, false, 1, false>(recs + q * MLORA_SMALL_TILE_WORDS, 0, 1, R, sp, y_col0, y_col1, y_col2, slice, xv, yv_, xs, ys,
                                                   num_slots, scaling, eff_rank, check, plan_hdr, xc, s_red, s_hi, s_lo, s_stage, &s_ok);
  }
}

struct Launch {
  const MloraAddArgs* a;
  dim3 grid;
  uint32_t packed;
  int widest;
  int spin_ticks, trusted;
};

// Offsets of slice i's A and B from slice 0's, in units of 16 bytes, when they fit 40 bits.
bool offsets16(const MloraAddArgs* a, int i, long long* ao, long long* bo) {
  const long long da = static_cast<const char*>(a->slices[i].a) - static_cast<const char*>(a->slices[0].a);
  const long long db = static_cast<const char*>(a->slices[i].b) - static_cast<const char*>(a->slices[0].b);
  if ((da & 15) || (db & 15)) return false;
  const long long qa = da / 16, qb = db / 16, lim = 1ll << 39;
  if (qa < -lim || qa >= lim || qb < -lim || qb >= lim) return false;
  *ao = qa;
  *bo = qb;
  return true;
}

template <typename T, int R>
void launch_three(const MloraAddArgs* a, dim3 grid, int nt, int cum1, int cum2) {
  const PlanLayout lay = plan_layout(a->num_tokens, a->num_slots);
  long long o[4] = {0, 0, 0, 0};  // A of slices 1 and 2, B of slices 1 and 2
  (void)offsets16(a, 1, &o[0], &o[2]);
  (void)offsets16(a, 2, &o[1], &o[3]);
  const uint32_t ao1 = static_cast<uint32_t>(o[0]), ao2 = static_cast<uint32_t>(o[1]), bo1 = static_cast<uint32_t>(o[2]), bo2 = static_cast<uint32_t>(o[3]);
  uint32_t high = 0;
  for (int i = 0; i < 4; ++i) high |= static_cast<uint32_t>((o[i] >> 32) & 0xff) << (8 * i);
  const uint32_t w01 = static_cast<uint32_t>(a->slices[0].n / 8) | (static_cast<uint32_t>(a->slices[1].n / 8) << 16);
  const uint32_t w2 = static_cast<uint32_t>(a->slices[2].n / 8) | (static_cast<uint32_t>(cum1) << 16) | (static_cast<uint32_t>(cum2) << 24);
  const uint32_t packed = static_cast<uint32_t>(nt / 64) | (static_cast<uint32_t>(a->num_slots) << 16);
  const uint32_t check = static_cast<uint32_t>(MLORA_PLAN_CHECK(a->num_tokens, a->num_slots));
  if (a->effective_rank)
    hipLaunchKernelGGL((slot_kernel3<T, R, true>), grid, dim3(kNW * kWave), 0, static_cast<hipStream_t>(a->stream), a->plan + lay.slotrec_off,
                       a->slices[0].a, a->slices[0].b, ao1, ao2, bo1, bo2, high, w01, w2, packed, a->x, a->y, a->x_stride, a->y_stride,
                       a->slices[0].y_col, a->slices[1].y_col, a->slices[2].y_col, check, a->scaling, a->effective_rank,
                       const_cast<int32_t*>(a->plan));
  else
    hipLaunchKernelGGL((slot_kernel3<T, R, false>), grid, dim3(kNW * kWave), 0, static_cast<hipStream_t>(a->stream), a->plan + lay.slotrec_off,
                       a->slices[0].a, a->slices[0].b, ao1, ao2, bo1, bo2, high, w01, w2, packed, a->x, a->y, a->x_stride, a->y_stride,
                       a->slices[0].y_col, a->slices[1].y_col, a->slices[2].y_col, check, a->scaling, a->effective_rank,
                       const_cast<int32_t*>(a->plan));
}

template <typename T, int R, int KSPW, int KP, bool MASKED, bool GR, int SA>
void launch_spans(const Launch& l) {
  const MloraAddArgs* a = l.a;
  const PlanLayout lay = plan_layout(a->num_tokens, a->num_slots);
  const MloraSlice& s0 = a->slices[0];
  const MloraSlice s1 = a->num_slices > 1 ? a->slices[1] : MloraSlice{nullptr, nullptr, 0, 0};
  hipLaunchKernelGGL((slot_kernel<T, R, KSPW, KP, MASKED, GR, SA>), l.grid, dim3(kNW * kWave), 0, static_cast<hipStream_t>(a->stream),
                     a->plan + lay.slotrec_off, s0.a, s0.b, s1.a, s1.b, s0.n, s1.n, l.packed, a->r, a->x, a->y, a->x_stride, a->y_stride,
                     s0.y_col, s1.y_col, static_cast<uint32_t>(MLORA_PLAN_CHECK(a->num_tokens, a->num_slots)), a->scaling,
                     a->effective_rank, const_cast<int32_t*>(a->plan), static_cast<uint32_t*>(a->workspace), l.spin_ticks, l.trusted);
}

template <typename T, int R, int KSPW, int KP>
void launch_one(const Launch& l) {
  if constexpr (R >= 32) {
    if (l.a->r != R) {  // buffers of a rank between the instances': the masked code with the buffers' rank as stride
      if (l.widest <= kNW * 64) launch_spans<T, R, KSPW, KP, true, true, 1>(l);
      else launch_spans<T, R, KSPW, KP, true, true, 2>(l);
      return;
    }
  }
  if (l.a->effective_rank) {
    if (l.widest <= kNW * 64) launch_spans<T, R, KSPW, KP, true, false, 1>(l);
    else launch_spans<T, R, KSPW, KP, true, false, 2>(l);
  } else {
    if (l.widest <= kNW * 64) launch_spans<T, R, KSPW, KP, false, false, 1>(l);
    else launch_spans<T, R, KSPW, KP, false, false, 2>(l);
  }
}

// kp: K parts (1: every workgroup multiplies the whole of K).
template <typename T>
bool launch_rank(const Launch& l, int rank, int kspw, int kp) {
  const int r = compute_rank(rank);
  if (kspw == 4 && kp == 1) {
    switch (r) {
      case 8: launch_one<T, 8, 4, 1>(l); return true;
      case 16: launch_one<T, 16, 4, 1>(l); return true;
      case 32: launch_one<T, 32, 4, 1>(l); return true;
      case 64: launch_one<T, 64, 4, 1>(l); return true;
    }
  } else if (kspw == 4 && kp == 4) {
    switch (r) {
      case 8: launch_one<T, 8, 4, 4>(l); return true;
      case 16: launch_one<T, 16, 4, 4>(l); return true;
      case 32: launch_one<T, 32, 4, 4>(l); return true;
      case 64: launch_one<T, 64, 4, 4>(l); return true;
    }
  } else if (kspw == 16 && kp == 1) {
    switch (r) {
      case 8: launch_one<T, 8, 16, 1>(l); return true;
      case 16: launch_one<T, 16, 16, 1>(l); return true;
    }
  }
  return false;
}

// Columns per range: as in the tile-major launch, sized for 150-250 workgroups; at most 1024 (two
// 64-column spans per wavefront, all loads in registers).
int range_columns(const MloraAddArgs* a) {
  long long cols = 0;
  for (int i = 0; i < a->num_slices; ++i) cols += a->slices[i].n;
  const int segs = a->num_slots < a->num_tokens ? a->num_slots : a->num_tokens;
  const int by_tokens = (a->num_tokens + MLORA_TILE_SMALL - 1) / MLORA_TILE_SMALL;
  const long long tiles = segs > by_tokens ? segs : by_tokens;  // about the number of tiles in use
  int nt = static_cast<int>(cols * tiles / 160);
  if (nt > 1024) nt = 1024;
  if (nt < 128) nt = 128;
  nt = (nt + 63) & ~63;
  while (nt < 1024) {
    int total = 0;
    for (int i = 0; i < a->num_slices; ++i) total += (a->slices[i].n + nt - 1) / nt;
    if (total <= 32) break;
    nt *= 2;
  }
  return nt > 1024 ? 1024 : nt;
}

int kspw_of(const MloraAddArgs* a) { return a->k % (32 * kNW) == 0 ? a->k / (32 * kNW) : 0; }

// Diagnostic knobs, read from the environment once per process.
struct SlotKnobs {
  int generation = -1, kparts, spin_ticks;
  void read() {
    generation = knob_generation();
    kparts = env_int("MLORA_SLOT_KPARTS", 4);          // 1: never share K out between workgroups
    spin_ticks = env_int("MLORA_SLOT_SPIN_TICKS", 20000);  // 200 us; 0: do not wait; < 0: never accept a partner's words
  }
};
SlotKnobs& slot_knobs() {
  static SlotKnobs k;
  if (k.generation != knob_generation()) k.read();
  return k;
}

// K parts of a launch: four for K = 4096 when the tile's workgroups can hand each other partial
// sums (one slice of at most 4096 columns, a workspace whose exchange area holds every tile's parts),
// else one.
int k_parts(const MloraAddArgs* a) {
  if (a->k != 4096 || a->num_slices != 1 || slot_knobs().kparts != 4) return 1;
  if (a->slices[0].n > 4 * 1024 || a->slices[0].n < 4 * 64) return 1;
  if (a->r > 32 && a->slices[0].n > 4 * 512) return 1;  // (two spans per wavefront at rank 64 do not fit the registers beside the parts)
  if (!a->workspace || (reinterpret_cast<uintptr_t>(a->workspace) & 255) || a->workspace_bytes < MLORA_WORKSPACE_HEAD_BYTES) return 1;
  const PlanLayout lay = plan_layout(a->num_tokens, a->num_slots);
  const long long words = static_cast<long long>(lay.cap_slotrec + lay.cap_over) * 4 * ((compute_rank(a->r) + 15) / 16) * 256;
  if (words * 8 > kWsXchgBytes) return 1;
  return 4;
}

}  // namespace

// K = 1024 at every rank; K = 4096 at every rank with the K parts of a tile shared out between its
// workgroups, else up to rank 16 (what fits the register file as one batch of loads); one or two
// slices with their pointers as arguments, three (K = 1024) with the later two's as offsets from
// the first one's; 16-bit elements.
bool slot_supported(const MloraAddArgs* a) {
  if (a->dtype != MLORA_DTYPE_BF16 && a->dtype != MLORA_DTYPE_F16) return false;
  if (a->num_slices < 1 || a->num_slices > 3 || !a->plan) return false;
  long long cols = 0;
  for (int i = 0; i < a->num_slices; ++i) {
    if (a->slices[i].n <= 0) return false;
    cols += a->slices[i].n;
  }
  if (cols > 200 * 1024) return false;  // at most 255 column ranges of up to 1024 columns
  if (!padded_rank(a->r)) return false;
  const int kspw = kspw_of(a);
  if (a->num_slices == 3) {
    // q | k | v: K = 1024, an exact rank, offsets that fit 40 bits, widths that fit 16-bit counts of
    // eight columns, and column ranges of at most 512 columns (one span per wavefront)
    long long ao, bo;
    if (kspw != 4 || !exact_rank(a->r) || !offsets16(a, 1, &ao, &bo) || !offsets16(a, 2, &ao, &bo)) return false;
    for (int i = 0; i < 3; ++i)
      if (a->slices[i].n % 8 || a->slices[i].n / 8 > 0xffff) return false;
    return range_columns(a) <= kNW * 64;
  }
  if (kspw == 4) return true;
  if (kspw == 16) return a->r <= 16 || k_parts(a) == 4;
  return false;
}

int slot_k_parts(const MloraAddArgs* a) { return k_parts(a); }

void slot_trace_set(void* buf) {
#ifdef MLORA_TRACE
  (void)hipMemcpyToSymbol(HIP_SYMBOL(trace_buf), &buf, sizeof(buf));
#else
  (void)buf;
#endif
}

int launch_slot(const MloraAddArgs* a, bool trusted_workspace) {
  const PlanLayout lay = plan_layout(a->num_tokens, a->num_slots);
  const int kp = k_parts(a);
  // with K parts the tile's workgroups are its K parts and its column ranges alike
  const int nt = kp > 1 ? ((a->slices[0].n + kp - 1) / kp + 63) & ~63 : range_columns(a);
  const int ranges0 = kp > 1 ? kp : (a->slices[0].n + nt - 1) / nt;
  const int ranges1 = a->num_slices > 1 ? (a->slices[1].n + nt - 1) / nt : 0;
  const int total = ranges0 + ranges1 + (a->num_slices > 2 ? (a->slices[2].n + nt - 1) / nt : 0);
  if (total > 255) {
    set_error("mlora_add_lora(slot-major): %d column ranges exceed 255", total);
    return MLORA_E_UNSUPPORTED;
  }
  Launch l;
  l.a = a;
  l.packed = static_cast<uint32_t>(nt / 64) | (static_cast<uint32_t>(ranges0) << 8) | (static_cast<uint32_t>(a->num_slots) << 16);
  l.widest = 0;
  for (int i = 0; i < a->num_slices; ++i) {
    const int w = a->slices[i].n < nt ? a->slices[i].n : nt;
    if (w > l.widest) l.widest = w;
  }
  l.spin_ticks = slot_knobs().spin_ticks;
  l.trusted = trusted_workspace ? 1 : 0;
  l.grid = dim3(8, static_cast<unsigned>(total), static_cast<unsigned>((lay.cap_slotrec + lay.cap_over) / 8));
  if (a->num_slices == 3) {
    switch (a->r) {
#define MLORA_THREE(R)                                                                                      \
  case R:                                                                                                   \
    if (a->dtype == MLORA_DTYPE_BF16) launch_three<__bf16, R>(a, l.grid, nt, ranges0, ranges0 + ranges1);   \
    else launch_three<_Float16, R>(a, l.grid, nt, ranges0, ranges0 + ranges1);                              \
    break;
      MLORA_THREE(8)
      MLORA_THREE(16)
      MLORA_THREE(32)
      MLORA_THREE(64)
#undef MLORA_THREE
      default: set_error("mlora_add_lora(slot-major): unsupported rank %d for three slices", a->r); return MLORA_E_UNSUPPORTED;
    }
    return check_launch("mlora_add_lora(small tiles, one workgroup per slot and column range, three slices)");
  }
  const int kspw = kspw_of(a) / kp;
  const bool ok = a->dtype == MLORA_DTYPE_BF16 ? launch_rank<__bf16>(l, a->r, kspw, kp) : launch_rank<_Float16>(l, a->r, kspw, kp);
  if (!ok) {
    set_error("mlora_add_lora(slot-major): unsupported rank %d / K %d", a->r, a->k);
    return MLORA_E_UNSUPPORTED;
  }
  return check_launch("mlora_add_lora(small tiles, one workgroup per slot and column range)");
}

}  // namespace mlora
