// Computes, for decode-sized batches, what the reference computes with a shrink launch, a
// temporary [slices, T, r] tensor and one or two expand launches
// (nanovllm_voxcpm/lora.py:291-381 driving lora_ops/triton_ops/lora_shrink_op.py:16-173,
// lora_expand_op.py:11-91 and kernel_utils.py:7-228; its small-batch dispatch:
// lora_shrink_op.py:10-13, 176-210): y_i[t] += (x[t] . A_i[s_t]^T) . B_i[s_t]^T * scaling.
//
// Small-tile form: one workgroup per (small tile, slice, column range).  A small tile is up
// to sixteen tokens of one slot, described by a self-contained 128-byte record.
//
// A launch of this size (a few MB) is bound by fixed latencies and by how fast one compute
// unit takes data in (about 20 bytes per cycle, cache-resident or not), not by HBM bandwidth,
// so the kernel is built around the number of dependent round trips to memory and the launch
// around the number of workgroups:
//   0. the scalar launch arguments arrive preloaded in SGPRs (the kernel takes them as plain
//      leading arguments for that purpose), so no fetch of the argument block comes first;
//   1. the plan header, the tile record, the token indices and the column-range entry are
//      fetched together — their addresses depend on nothing but the workgroup index — and one
//      branch-free test decides whether the workgroup has work;
//   2. every global load the workgroup needs — its K-range of the x rows and of A[slot], the
//      B[slot] rows and the y rows of its output spans — is issued before any arithmetic;
//   3. column ranges are sized on the host so that a launch spreads over 150-250 workgroups.
// Both products run on the matrix cores (v_mfma_f32_16x16x32, fp32 accumulate): the sixteen
// token rows are one MFMA dimension, so a half-empty tile costs nothing but idle multiplier
// lanes.  The eight wavefronts split K for the shrink, sum their partial tiles through LDS,
// keep the rank-r intermediate there as a hi + lo pair of operand-precision values, and then
// each take 64-column spans of the expand; the B rows of a span are interleaved across its
// four MFMAs so that a lane owns consecutive columns and y is updated with wide accesses.
#include "common.h"
#include "launch.h"

namespace mlora {

namespace {

constexpr int kMaxSplits = 32;
constexpr int kNW = 8;          // wavefronts per workgroup
constexpr int kSpansAheadMax = 2;  // output spans per wavefront whose loads are issued up front (SA: 1 or 2)

MLORA_TRACE_DECL

struct DecodeSplit {
  const void* a;
  const void* b;
  int n, y_col, n0, n1;
};

struct DecodeSplits {
  DecodeSplit split[kMaxSplits];
};

// KSPW: k-steps (32 elements of K) each wavefront covers when that is known at compile time
// (K = 32 * kNW * KSPW), 0 when it has to be worked out from K at run time.
//
// eff_rank (may be null): rank of the adapter resident in each slot.  16-rank blocks of A[slot] at
// or above it are neither fetched nor multiplied, the intermediate is zero from that rank on, and
// B[slot] elements from that rank on are replaced by zeros before they reach a multiplier.
//
// TR (KSPW a multiple of four): a compute unit's vector L1 handles a 128-bit load whose consecutive
// lanes touch different rows (what the MFMA operand layout asks for) at about a quarter of the
// rate of one whose lanes walk along a row, and even cache-resident operands showed up as
// 3-4 us per launch.  With TR the x rows and A rows of a wavefront's K range are fetched
// row-contiguously (sixteen lanes per 256 bytes of a row) and turned into operand layout through
// a private LDS block per wavefront, and the expand runs with the tokens as MFMA rows, so that
// sixteen consecutive lanes cover 128 contiguous bytes of one y row.
//
// SA: spans per wavefront requested up front.  A launch whose column ranges are at most 512 columns
// wide (one span per wavefront) takes the instance with SA = 1: the second span's requests, though
// clamped to a line or two, cost 0.2 us per launch (o 4.31 -> 4.07, qkv 4.44 -> 4.25, down 7.02 -> 6.81).
//
// GR (with MASKED): the buffers' rank is `rbuf_arg` < R, a multiple of eight (24 in the instance for
// 32; 40, 48, 56 in the one for 64): rows of A[slot] are rbuf * K apart, B rows rbuf elements long, and
// whatever lies beyond rbuf is treated like the ranks beyond an adapter's own (requests clamped
// into the buffers, values masked).
template <typename T, int R, int KSPW, bool TR, bool MASKED, int SA, bool GR = false>
__global__ __launch_bounds__(kNW* kWave) void decode_kernel(const int32_t* __restrict__ plan, const void* __restrict__ xv,
                                                            void* __restrict__ yv_, int64_t xs, int64_t ys, int small_off,
                                                            int include_long, int T_, int K, int num_slots, float scaling,
                                                            const int32_t* __restrict__ eff_rank, int rbuf_arg, DecodeSplits splits) {
  static_assert(!GR || (MASKED && R >= 32), "buffers of a rank between the instances' take the masked code of the next instance up");
  constexpr int RB = (R + 15) / 16;      // 16-rank blocks of the shrink output
  constexpr int KSTEPS = (R + 31) / 32;  // MFMA k-steps of the expand
  constexpr int HSTRIDE = R + 8;         // padded LDS row of the intermediate
  constexpr int NT = kNW * kWave;
  constexpr int CH = TR ? 4 : KSPW > 0 ? KSPW : 4;  // k-steps whose operands are in registers together
  constexpr int ROUNDS = TR ? KSPW / 4 : 1;          // staged form: groups of four k-steps per wavefront

  __shared__ __attribute__((aligned(16))) float s_red[kNW * RB * 64 * 4];
  __shared__ __attribute__((aligned(16))) T s_hi[16 * HSTRIDE];
  __shared__ __attribute__((aligned(16))) T s_lo[16 * HSTRIDE];
  constexpr int kStageRow = 17;  // 16 chunks of 16 bytes + one of padding: operand reads hit every bank once
  constexpr int SB = RB < 2 ? RB : 2;  // 16-rank blocks of A staged together (rank 64 goes through in two passes)
  __shared__ __attribute__((aligned(16))) i32x4 s_stage[TR ? kNW * (1 + SB) * 16 * kStageRow : 1];
  static_assert(!TR || (KSPW >= 4 && KSPW % 4 == 0), "the staged form takes the k-steps of a wavefront four at a time");

  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int lr = lane & 15, lg = lane >> 4;
  const int rbuf = GR ? rbuf_arg : R;  // rank of the buffers: row count of A[slot], row length of B
  MLORA_STAMP(0);  // first instruction

  // grid (8, column ranges, tiles / 8): linear workgroup ids advance along x first and
  // consecutive ids go to consecutive XCDs, so blockIdx.x is the XCD: the column ranges of one
  // tile share an XCD and its L2.
  const int split_id = blockIdx.y;
  const int tile = blockIdx.z * 8 + blockIdx.x;

  // ---- round trip 1 ---------------------------------------------------------------------------
  const int32_t* rec = plan + small_off + tile * MLORA_SMALL_TILE_WORDS;  // tile < capacity: in bounds
  const int row = rec[MLORA_SMALL_TILE_ROWS + lr];
  const i32x4 rows4 = *reinterpret_cast<const i32x4*>(rec + MLORA_SMALL_TILE_ROWS + 4 * lg);  // tokens 4*lg .. 4*lg+3
  const i32x4 rec0 = *reinterpret_cast<const i32x4*>(rec);       // slot, count, start, 0
  typedef int i32x16 __attribute__((ext_vector_type(16)));
  const DecodeSplit sp = splits.split[split_id];
  const i32x16 hdr = *reinterpret_cast<const i32x16*>(plan);  // the whole header in one scalar load
  const RankPrefetch ranks = rank_prefetch(MASKED ? eff_rank : nullptr, num_slots, lane);
  // (everything above is requested before anything below is scheduled: left to itself the
  // compiler requests this launch's column range only after the header has arrived)
  __builtin_amdgcn_sched_barrier(0);
  const int slot = rec0[0], m = rec0[1];
  const int n_tiles = hdr[MLORA_PLAN_TILES_SHORT] + hdr[MLORA_PLAN_TILES_LONG_SMALL] * include_long;
  // One exit test, evaluated without short-circuit, that consumes everything fetched above
  // (the token index through its first lane), so that all of it is requested here, together,
  // instead of piece by piece behind a chain of branches.
  const int usable = int(hdr[MLORA_PLAN_MAGIC] == MLORA_PLAN_MAGIC_VALUE) & int(hdr[MLORA_PLAN_NUM_TOKENS] == T_) &
                     int(hdr[MLORA_PLAN_MAX_SLOTS] == num_slots) & int(tile < n_tiles) & int(m > 0) &
                     int(slot < num_slots) & int(sp.n0 < sp.n1) & int(sp.a != nullptr) & int(sp.b != nullptr) &
                     int(sp.n > 0) & int(sp.y_col >= 0) & int(__builtin_amdgcn_readfirstlane(row) >= 0) &
                     int(__builtin_amdgcn_readfirstlane(rows4[0]) >= 0);
  if (!usable) {
    count_rejected_plan(plan, hdr[MLORA_PLAN_MAGIC] == MLORA_PLAN_MAGIC_VALUE && hdr[MLORA_PLAN_NUM_TOKENS] == T_ &&
                                  hdr[MLORA_PLAN_MAX_SLOTS] == num_slots);
    return;
  }
  MLORA_STAMP(1);  // tile record and plan header are here

  // rank of the adapter in this slot (requested together with the record, see rank_prefetch)
  // (MASKED = false is the instance for callers that gave no rank vector: eff is the constant R
  // there and every test on it below folds away)
  int eff = MASKED ? rank_pick(ranks, eff_rank, num_slots, slot, R) : R;
  if (GR && eff > rbuf) eff = rbuf;
  if (MASKED && eff == 0) return;
  const int rb_n = MASKED ? (eff + 15) >> 4 : RB;  // 16-rank blocks of A in use

  const bool live = lr < m;  // this lane's token exists
  const T* xrow = static_cast<const T*>(xv) + static_cast<int64_t>(row) * xs + lg * 8;
  const T* A = static_cast<const T*>(sp.a) + static_cast<int64_t>(slot) * rbuf * K;
  const T* arow[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int rr = rb * 16 + lr;
    arow[rb] = A + static_cast<int64_t>(rr < rbuf ? rr : rbuf - 1) * K + lg * 8;
  }
  const T* B = static_cast<const T*>(sp.b) + static_cast<int64_t>(slot) * sp.n * rbuf;
  T* yrow = static_cast<T*>(yv_) + static_cast<int64_t>(row) * ys + sp.y_col + 16 * lg;

  // ---- round trip 2: issue every load ---------------------------------------------------------
  const int nks = K / 32;  // k-steps of the contraction
  const int ks0 = KSPW > 0 ? wave * KSPW : wave * nks / kNW;
  const int ks1 = KSPW > 0 ? ks0 + KSPW : (wave + 1) * nks / kNW;
  Pack8 xa[CH], aw[RB][CH];
  i32x4 xst[TR ? 4 * ROUNDS : 1], ast[TR ? RB : 1][TR ? 4 * ROUNDS : 1];
  if constexpr (TR) {
    // row-contiguous: lane = (row group lane/16, 16-byte chunk lane%16 of a 256-byte K range);
    // one such range (four k-steps) per round
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) {
      const int64_t koff = static_cast<int64_t>(ks0 + 4 * r) * 32 + (lane & 15) * 8;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        xst[4 * r + i] = load128(static_cast<const T*>(xv) + static_cast<int64_t>(rows4[i]) * xs + koff);
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
          const int rr = rb * 16 + 4 * lg + i;
          if (!MASKED || RB == 1 || rb < rb_n) ast[rb][4 * r + i] = load128(A + static_cast<int64_t>(rr < rbuf ? rr : rbuf - 1) * K + koff);
          else ast[rb][4 * r + i] = i32x4{0, 0, 0, 0};
        }
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int ks = ks0 + i;
      if (KSPW > 0 || ks < ks1) {
        xa[i].raw = load128(xrow + ks * 32);  // absent tokens read row 0; their results are never stored
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) aw[rb][i].raw = load128(arow[rb] + ks * 32);
      }
    }
  }
  constexpr int kSpansAhead = SA;
  Pack8 bop[kSpansAhead][4][KSTEPS], yreg[kSpansAhead][2];
  uint2 yq[TR ? kSpansAhead : 1][TR ? 4 : 1];  // TR: four columns of four tokens per lane and span
  T* const ycols = static_cast<T*>(yv_) + sp.y_col;
  // TR span: MFMA j takes column c0 + 4 * (lane % 16) + j, so a lane ends up with four consecutive
  // columns of tokens 4 * (lane / 16) .. + 3
  constexpr bool K16 = TR && R == 16;  // expand on the 16x16x16 MFMA: 64-bit operand pieces
  auto load_span_tr = [&](int c0, Pack8(&bo)[4][KSTEPS], uint2(&yy)[4]) {
    if constexpr (K16) {
      // A span's 64 B rows of 32 bytes are 2 KB of contiguous memory: fetched as such (lane l takes
      // 16 bytes of row c0 + l / 2 and of row c0 + 32 + l / 2, eight cache lines per instruction
      // instead of sixteen quarter-used ones); finish_span_tr turns them into operand pieces.
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        int n = c0 + 32 * h + (lane >> 1);
        n = n < sp.n1 ? n : sp.n1 - 1;
        bo[h][0].raw = load128(B + static_cast<int64_t>(n) * R + (lane & 1) * 8);
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
          bo[j][ks].raw = load128(B + static_cast<int64_t>(n) * rbuf + kc * 8);
        }
      }
    }
    const int c = c0 + 4 * lr < sp.n1 ? c0 + 4 * lr : sp.n1 - 4;
#pragma unroll
    for (int i = 0; i < 4; ++i) yy[i] = *reinterpret_cast<const uint2*>(ycols + static_cast<int64_t>(rows4[i]) * ys + c);
  };
#pragma unroll
  for (int s = 0; s < kSpansAhead; ++s) {
    const int c0 = sp.n0 + (wave + s * kNW) * 64;
    if constexpr (TR) {
      // requested whether the span exists or not (the addresses of one that does not are clamped
      // into the range: a cache line or two, never stored): values that are requested in a branch
      // and used in a later one are unpacked by the compiler where they are requested, and the
      // wavefront then waits for them before it has requested anything else
      load_span_tr(c0, bop[s], yq[s]);
    } else if (c0 < sp.n1) {
      {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          int n = c0 + 16 * (lr >> 2) + 4 * j + (lr & 3);
          n = n < sp.n1 ? n : sp.n1 - 1;
#pragma unroll
          for (int ks = 0; ks < KSTEPS; ++ks) {
            // lanes whose chunk lies beyond the rank fetch a valid chunk anyway: their H operand is
            // zero, and an unconditional load keeps the whole batch of loads in flight together
            int kc = (lg + 4 * ks) & (R / 8 - 1);
            if (GR && kc * 8 >= rbuf) kc = rbuf / 8 - 1;  // (masked where it is used)
            bop[s][j][ks].raw = load128(B + static_cast<int64_t>(n) * rbuf + kc * 8);
          }
        }
#pragma unroll
        for (int half = 0; half < 2; ++half)
          if (live && c0 + 16 * lg + 8 * half < sp.n1) yreg[s][half].raw = load128(yrow + c0 + 8 * half);
      }
    }
  }

  MLORA_STAMP(2);  // every load is issued
  // ---- shrink: H[token, rank] partial over this wavefront's K range ----------------------------
  f32x4 acc[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) acc[rb] = f32x4{0.f, 0.f, 0.f, 0.f};
  if constexpr (TR) {
    // through the wavefront's LDS block: written row-contiguously, read in operand layout
    // (k-step i of lane group g is chunk 4 * i + g, the same elements the direct loads take)
    i32x4* stage = s_stage + wave * (1 + SB) * 16 * kStageRow;
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) {
#pragma unroll
      for (int i = 0; i < 4; ++i) stage[(4 * lg + i) * kStageRow + (lane & 15)] = xst[4 * r + i];
#pragma unroll
      for (int p = 0; p < RB / SB; ++p) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
#pragma unroll
          for (int sb = 0; sb < SB; ++sb) stage[((1 + sb) * 16 + 4 * lg + i) * kStageRow + (lane & 15)] = ast[p * SB + sb][4 * r + i];
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
      // this round's k-steps, in ascending order as the direct form takes them
#pragma unroll
      for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) acc[rb] = Mma<T>::run(xa[i], aw[rb][i], acc[rb]);
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      if (KSPW > 0 || ks0 + i < ks1) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) acc[rb] = Mma<T>::run(xa[i], aw[rb][i], acc[rb]);
      }
    }
  }
  if (KSPW == 0) {
    for (int ksb = ks0 + CH; ksb < ks1; ksb += CH) {  // K not known at compile time: further batches
#pragma unroll
      for (int i = 0; i < CH; ++i) {
        const int ks = ksb + i;
        if (ks < ks1) {
          xa[i].raw = load128(xrow + ks * 32);
#pragma unroll
          for (int rb = 0; rb < RB; ++rb) aw[rb][i].raw = load128(arow[rb] + ks * 32);
        }
      }
#pragma unroll
      for (int i = 0; i < CH; ++i) {
        if (ksb + i < ks1) {
#pragma unroll
          for (int rb = 0; rb < RB; ++rb) acc[rb] = Mma<T>::run(xa[i], aw[rb][i], acc[rb]);
        }
      }
    }
  }

  // Sum the K-partials of the wavefronts.  D layout: lane holds H[token 4*(lane/16)+i][rank lane%16].
  if constexpr (KSPW == 0) mfma_settle(acc);  // k-steps past the end of K were skipped by branches
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) *reinterpret_cast<f32x4*>(&s_red[((wave * RB + rb) * 64 + lane) * 4]) = acc[rb];
  MLORA_STAMP(3);  // wavefront 0: x and A arrived, staged and multiplied
  __syncthreads();
  MLORA_STAMP(4);  // every wavefront's partial is in LDS
  for (int e = tid; e < RB * 256; e += NT) {
    const int rb = e >> 8, ln = (e & 255) >> 2, i = e & 3;
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < kNW; ++w) sum += s_red[((w * RB + rb) * 64 + ln) * 4 + i];
    const int tok = 4 * (ln >> 4) + i, r = rb * 16 + (ln & 15);
    if (r < R) {
      const float v = (!MASKED || r < eff) ? sum * scaling : 0.f;  // ranks the adapter does not have contribute nothing
      const T hi = from_f32<T>(v);
      s_hi[tok * HSTRIDE + r] = hi;
      s_lo[tok * HSTRIDE + r] = from_f32<T>(v - to_f32(hi));
    }
  }
  __syncthreads();
  MLORA_STAMP(5);  // the intermediate is in LDS

  // ---- expand ---------------------------------------------------------------------------------
  Pack8 hop[KSTEPS], hlo[KSTEPS];
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

  // Ranks at or above the adapter's are cleared in the B operands where they are used, not where
  // they were requested: cleared at the request, every load is waited for on the spot.
  auto mask_b = [&](Pack8(&bo)[4][KSTEPS]) {
    if (MASKED && eff < R) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) mask_ranks(bo[j][ks], ((lg + 4 * ks) & (R / 8 - 1)) * 8, eff);
    }
  };
  auto finish_span = [&](int c0, Pack8(&bo)[4][KSTEPS], Pack8(&yy)[2]) {
    f32x4 out[4];
    mask_b(bo);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      out[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        out[j] = Mma<T>::run(bo[j][ks], hlo[ks], out[j]);
        out[j] = Mma<T>::run(bo[j][ks], hop[ks], out[j]);
      }
    }
    if (live) {
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        if (c0 + 16 * lg + 8 * half < sp.n1) {
          float yf[8];
          unpack8<T>(yy[half], yf);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            yf[i] += out[2 * half][i];
            yf[4 + i] += out[2 * half + 1][i];
          }
          Pack8 r;
          pack8<T>(yf, r);
          store128(yrow + c0 + 8 * half, r.raw);
        }
      }
    }
  };
  // tokens as MFMA rows: lane holds out[token 4 * lg + i][column c0 + 4 * lr + j]
  uint2 hop16 = {0, 0}, hlo16 = {0, 0};
  if constexpr (K16) {
    hop16 = *reinterpret_cast<const uint2*>(&s_hi[lr * HSTRIDE + 4 * lg]);
    hlo16 = *reinterpret_cast<const uint2*>(&s_lo[lr * HSTRIDE + 4 * lg]);
  }
  auto finish_span_tr = [&](int c0, Pack8(&bo)[4][KSTEPS], uint2(&yy)[4]) {
    f32x4 out[4];
    uint2 pieces[4];
    if constexpr (K16) {
      if (MASKED && eff < R) {
        mask_ranks(bo[0][0], (lane & 1) * 8, eff);
        mask_ranks(bo[1][0], (lane & 1) * 8, eff);
      }
      // B rows -> operand pieces through the wavefront's LDS block: four rows (128 bytes) per
      // group, groups 144 bytes apart so that the sixteen lanes of a piece read hit every bank
      // once.  MFMA j of lane (lr, lg) takes ranks 4*lg .. 4*lg+3 of column c0 + 4*lr + j.
      char* blk = reinterpret_cast<char*>(s_stage + wave * (1 + SB) * 16 * kStageRow);
      *reinterpret_cast<i32x4*>(blk + (lane >> 3) * 144 + (lane & 7) * 16) = bo[0][0].raw;
      *reinterpret_cast<i32x4*>(blk + ((lane >> 3) + 8) * 144 + (lane & 7) * 16) = bo[1][0].raw;
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int j = 0; j < 4; ++j) pieces[j] = *reinterpret_cast<const uint2*>(blk + lr * 144 + j * 32 + lg * 8);
      __builtin_amdgcn_wave_barrier();
    } else {
      mask_b(bo);
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
    // (the y values are taken as they are only here: left to itself the compiler unpacks them
    // where they were requested, and the wavefront then waits for their arrival before it has
    // requested its other spans and before the shrink)
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
  for (int s = 0; s < kSpansAhead; ++s) {
    const int c0 = sp.n0 + (wave + s * kNW) * 64;
    if (c0 < sp.n1) {
      if constexpr (TR) finish_span_tr(c0, bop[s], yq[s]);
      else finish_span(c0, bop[s], yreg[s]);
    }
  }
  MLORA_STAMP(6);  // wavefront 0: its first spans are multiplied and their stores issued
  for (int c0 = sp.n0 + (wave + kSpansAhead * kNW) * 64; c0 < sp.n1; c0 += kNW * 64) {  // wide ranges
    Pack8 bo[4][KSTEPS], yy[2];
    if constexpr (TR) {
      uint2 yt[4];
      load_span_tr(c0, bo, yt);
      finish_span_tr(c0, bo, yt);
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        int n = c0 + 16 * (lr >> 2) + 4 * j + (lr & 3);
        n = n < sp.n1 ? n : sp.n1 - 1;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
          int kc = (lg + 4 * ks) & (R / 8 - 1);
          if (GR && kc * 8 >= rbuf) kc = rbuf / 8 - 1;  // (masked where it is used)
          bo[j][ks].raw = load128(B + static_cast<int64_t>(n) * rbuf + kc * 8);
        }
      }
#pragma unroll
      for (int half = 0; half < 2; ++half)
        if (live && c0 + 16 * lg + 8 * half < sp.n1) yy[half].raw = load128(yrow + c0 + 8 * half);
      finish_span(c0, bo, yy);
    }
  }
#ifdef MLORA_TRACE
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  MLORA_STAMP(7);  // wavefront 0: its stores are acknowledged
  __syncthreads();
  MLORA_STAMP(8);  // every wavefront is done
#endif
}

struct Launch {
  const MloraAddArgs* a;
  int small_off, include_long, staged;
  int widest;  // columns of the widest column range
  dim3 grid;
  const DecodeSplits* splits;
};

template <typename T, int R, int KSPW, bool TR, bool MASKED, int SA, bool GR = false>
void launch_spans(const Launch& l) {
  const MloraAddArgs* a = l.a;
  hipLaunchKernelGGL((decode_kernel<T, R, KSPW, TR, MASKED, SA, GR>), l.grid, dim3(kNW * kWave), 0, static_cast<hipStream_t>(a->stream),
                     a->plan, a->x, a->y, a->x_stride, a->y_stride, l.small_off, l.include_long, a->num_tokens, a->k,
                     a->num_slots, a->scaling, a->effective_rank, a->r, *l.splits);
}

// One span per wavefront up front when no column range holds more (staged form; the other form
// keeps its two).
template <typename T, int R, int KSPW, bool TR, bool MASKED>
void launch_masked(const Launch& l) {
  if constexpr (TR) {
    if (l.widest <= kNW * 64) return launch_spans<T, R, KSPW, TR, MASKED, 1>(l);
  }
  launch_spans<T, R, KSPW, TR, MASKED, kSpansAheadMax>(l);
}

// With a rank vector the instance that reads it; without, the one that has no such code at all.
template <typename T, int R, int KSPW, bool TR = false>
void launch_one(const Launch& l) {
  if (l.a->effective_rank) launch_masked<T, R, KSPW, TR, true>(l);
  else launch_masked<T, R, KSPW, TR, false>(l);
}

// The steps-per-wavefront specialisations kept: 1, 2 and 4 (K = 256, 512, 1024) for every rank
// and 16 (K = 4096) where the loads of sixteen steps still fit the register file.
template <typename T, int R>
void launch_kspw(const Launch& l, int kspw) {
  if constexpr (R >= 32) {
    if (l.a->r != R) {
      // buffers of a rank between the instances' (24; 40, 48, 56): the masked code of this instance
      // with the buffers' rank as stride, in the staged form for K = 1024 and the general one else
      if (l.staged && kspw == 4) {
        if (l.widest <= kNW * 64) return launch_spans<T, R, 4, true, true, 1, true>(l);
        return launch_spans<T, R, 4, true, true, kSpansAheadMax, true>(l);
      }
      return launch_spans<T, R, 0, false, true, kSpansAheadMax, true>(l);
    }
  }
  if (l.staged) {
    // staged operands, the k-steps of a wavefront four at a time (rank 64 in two passes of 32 ranks
    // through the same LDS block); how many k-steps fit is a matter of registers: every load of
    // the workgroup's K range is issued before the first is used
    if (kspw == 4) return launch_one<T, R, 4, true>(l);
    if constexpr (R <= 32) {
      if (kspw == 8) return launch_one<T, R, 8, true>(l);
    }
    if constexpr (R <= 16) {
      if (kspw == 12) return launch_one<T, R, 12, true>(l);
      if (kspw == 16) return launch_one<T, R, 16, true>(l);
    }
  }
  if (kspw == 4) return launch_one<T, R, 4>(l);
  if (kspw == 2) return launch_one<T, R, 2>(l);
  if (kspw == 1) return launch_one<T, R, 1>(l);
  if constexpr (R <= 16) {
    if (kspw == 16) return launch_one<T, R, 16>(l);
  }
  launch_one<T, R, 0>(l);
}

template <typename T>
void launch_rank(const Launch& l, int r, int kspw) {
  switch (compute_rank(r)) {
    case 8: launch_kspw<T, 8>(l, kspw); break;
    case 16: launch_kspw<T, 16>(l, kspw); break;
    case 32: launch_kspw<T, 32>(l, kspw); break;
    default: launch_kspw<T, 64>(l, kspw); break;
  }
}

// Diagnostic knobs, read from the environment once per process.
struct DecodeKnobs {
  int generation = -1, staged, nt;
  void read() {
    generation = knob_generation();
    staged = env_int("MLORA_DECODE_STAGED", 1);
    nt = env_int("MLORA_DECODE_NT", 0);
  }
};

}  // namespace

// Nothing in the kernel limits the size of x or y.
bool decode_supported(const MloraAddArgs*) { return true; }

void decode_trace_set(void* buf) {
#ifdef MLORA_TRACE
  (void)hipMemcpyToSymbol(HIP_SYMBOL(trace_buf), &buf, sizeof(buf));
#else
  (void)buf;
#endif
}

int launch_decode(const MloraAddArgs* a, bool include_long) {
  static DecodeKnobs knobs;
  if (knobs.generation != knob_generation()) knobs.read();
  DecodeSplits splits;
  const PlanLayout lay = plan_layout(a->num_tokens, a->num_slots);
  int cap = lay.cap_small;
  if (!include_long) {  // a segment below the threshold is exactly one small tile
    const int segs = a->num_slots < a->num_tokens ? a->num_slots : a->num_tokens;
    if (segs < cap) cap = segs;
  }
  if (cap == 0) return 0;
  cap = (cap + 7) & ~7;

  Launch l;
  l.a = a; l.small_off = lay.small_off; l.include_long = include_long ? 1 : 0; l.splits = &splits;
  l.staged = knobs.staged;

  // Column range per workgroup.  Every range repeats the shrink of its tile, but a compute unit
  // takes in only 30-60 bytes per cycle even from the L2, so a launch is fastest when its
  // bytes are spread over 150-250 workgroups: ranges shrink down to 128 columns for narrow
  // projections and stay at 1024 (two 64-column spans per wavefront, all loads still in
  // registers) for wide ones.  Measured per launch at 32 tiles: o 6.2 us at 1024 columns,
  // 5.1 at 512, 4.7 at 256; gate_up 8.2 / 8.9 / 11.1.
  int nt = knobs.nt;
  if (nt <= 0) {
    long long cols = 0;
    for (int i = 0; i < a->num_slices; ++i) cols += a->slices[i].n;
    const int segs = a->num_slots < a->num_tokens ? a->num_slots : a->num_tokens;
    const int by_tokens = (a->num_tokens + MLORA_TILE_SMALL - 1) / MLORA_TILE_SMALL;
    const long long tiles = segs > by_tokens ? segs : by_tokens;  // about the number of tiles in use
    nt = static_cast<int>(cols * tiles / 160);
    if (nt > 1024) nt = 1024;
    if (nt < 128) nt = 128;
  }
  if (nt < 64) nt = 64;
  nt = (nt + 63) & ~63;
  int total = 0;
  for (;;) {
    total = 0;
    for (int i = 0; i < a->num_slices; ++i) total += (a->slices[i].n + nt - 1) / nt;
    if (total <= kMaxSplits) break;
    nt *= 2;
  }
  if (total == 0) return 0;
  int s = 0;
  l.widest = 0;
  for (int i = 0; i < a->num_slices; ++i) {
    const MloraSlice& sl = a->slices[i];
    for (int n0 = 0; n0 < sl.n; n0 += nt) {
      DecodeSplit& d = splits.split[s++];
      d.a = sl.a; d.b = sl.b; d.n = sl.n; d.y_col = sl.y_col;
      d.n0 = n0; d.n1 = n0 + nt < sl.n ? n0 + nt : sl.n;
      if (d.n1 - d.n0 > l.widest) l.widest = d.n1 - d.n0;
    }
  }
  for (; s < kMaxSplits; ++s) splits.split[s] = DecodeSplit{nullptr, nullptr, 0, 0, 0, 0};
  l.grid = dim3(8, static_cast<unsigned>(total), static_cast<unsigned>(cap / 8));
  const int nks = a->k / 32;
  const int kspw = (nks % kNW == 0) ? nks / kNW : 0;
  if (a->dtype == MLORA_DTYPE_BF16) launch_rank<__bf16>(l, a->r, kspw);
  else launch_rank<_Float16>(l, a->r, kspw);
  return check_launch("mlora_add_lora(small tiles, one workgroup per column range)");
}

}  // namespace mlora
