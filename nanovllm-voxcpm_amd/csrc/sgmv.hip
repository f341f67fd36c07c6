// Computes, for prefill-sized batches, what the reference computes with its segment-grouped
// shrink and expand kernels (nanovllm_voxcpm/lora_ops/triton_ops/lora_shrink_op.py:16-101, 257-341,
// lora_expand_op.py:11-170, kernel_utils.py:7-228, launched from nanovllm_voxcpm/lora.py:291-381):
// y_i[t] += (x[t] . A_i[s_t]^T) . B_i[s_t]^T * scaling, tokens grouped by slot.
//
// SGMV form for batches above the small-batch limit: two launches that meet in a small
// workspace, both on the matrix cores (v_mfma_f32_16x16x32 bf16 / f16, fp32 accumulate).  Work
// units are the 64-token tiles of the long segments and, behind them in the same grids, the
// short segments (one small-tile record each).
//
//   shrink — H^T[rank x tokens] = A[slot] . X_tile^T for a (tile, slice, K part).  What bounds
//            this product is the number of bytes a compute unit takes in (cache hits cost about
//            as much as misses: the limit is requests in flight), so each operand element is
//            fetched once per workgroup: the A[slot] slab of the workgroup's K part is copied to
//            LDS with row-contiguous 128-bit loads and shared by the four wavefronts, each of
//            which owns sixteen tokens of the tile and streams their x rows straight from global
//            memory into the MFMA operand layout, a whole batch of k-steps in flight at a time.
//            No wavefront shares a sum with another, so the accumulators go straight to the
//            workspace as fp32; when K is split across workgroups each part writes its own
//            partial.  For three or more slices one workgroup walks all of them with the x rows
//            it holds.
//   expand — OUT[tokens x cols] = H . B[slot]^T for a (group of tiles, column range).  The H
//            tiles are staged in LDS once (K partials summed, scaled, and split into a hi + lo
//            pair of operand-precision values, about 16 significant bits: the expand loses
//            nothing that would show after the final rounding of y).  A wavefront owns spans of
//            64 or 128 columns: it fetches the span's B rows once per slot, then for every tile
//            of the group the y rows of two or four 16-token blocks at a time, runs the MFMAs
//            and writes y back.  Tokens are the MFMA rows and the B rows fed to the MFMAs of a
//            span are interleaved, so a lane ends up with consecutive output columns of four
//            tokens and sixteen consecutive lanes cover a contiguous piece of one y row: y moves
//            in fully coalesced accesses with no transposition pass.
// Splitting the two products means no column range repeats the shrink of its tile, and each
// kernel keeps only its own operands in registers.
#include "common.h"
#include "launch.h"

namespace mlora {

namespace {

constexpr int kMaxSplits = 64;
constexpr int kExpandWaves = 4;
constexpr int kMaxKSplit = 4;  // most K parts the shrink ever uses (the workspace has room for them)

struct ShrinkSlices {
  const void* a[MLORA_MAX_SLICES];
};

struct ExpandSplit {
  const void* b;
  int n, y_col, n0, n1, slice, pad;
};

struct ExpandSplits {
  ExpandSplit split[kMaxSplits];
};

// A unit of work of either kernel: up to 64 tokens of one slot.  Workgroups below `big_cap` take
// the 64-token tiles of the long segments; the ones above take the short segments (fewer than
// sixteen tokens, one small-tile record each), so that one pair of launches covers the batch.
struct TileRef {
  int slot, start, m, ok;
};

__device__ __forceinline__ TileRef fetch_tile(const int32_t* __restrict__ plan, int big_off, int small_off, int big_cap, int tile,
                                              int T_, int num_slots) {
  // both candidate records and the header are requested together (every address is in bounds
  // for the whole grid); the choice between them costs no second round trip
  const int sidx = tile >= big_cap ? tile - big_cap : 0;
  const i32x4 big = reinterpret_cast<const i32x4*>(plan + big_off)[tile < big_cap ? tile : 0];
  const i32x4 small = *reinterpret_cast<const i32x4*>(plan + small_off + sidx * MLORA_SMALL_TILE_WORDS);
  const i32x4 hdr0 = *reinterpret_cast<const i32x4*>(plan);
  const i32x4 hdr1 = *reinterpret_cast<const i32x4*>(plan + 4);
  const i32x4 hdr2 = *reinterpret_cast<const i32x4*>(plan + 8);
  const bool is_big = tile < big_cap;
  TileRef t;
  t.slot = is_big ? big[0] : small[0];
  t.start = is_big ? big[1] : small[2];
  t.m = is_big ? big[2] : small[1];
  const int limit = is_big ? hdr2[MLORA_PLAN_TILES_LONG_BIG - 8] : hdr1[MLORA_PLAN_TILES_SHORT - 4];
  const int index = is_big ? tile : sidx;
  t.ok = int(hdr0[MLORA_PLAN_MAGIC] == MLORA_PLAN_MAGIC_VALUE) & int(hdr0[MLORA_PLAN_NUM_TOKENS] == T_) &
         int(hdr0[MLORA_PLAN_MAX_SLOTS] == num_slots) & int(index < limit) & int(t.m > 0) & int(t.slot >= 0) &
         int(t.slot < num_slots);
  return t;
}

// ---- shrink -------------------------------------------------------------------------------------
// grid (8, slices * K parts, tiles / 8), four wavefronts of sixteen tokens each.  The workgroup's
// K part is walked in x batches of XW columns (a wavefront holds the batch of its sixteen token
// rows in registers) and, inside a batch, in A slabs of KR columns that pass through LDS.  Both
// streams run one step ahead of the MFMAs: the next slab sits in registers and the next x batch
// is in flight while the current slab is multiplied, so that a compute unit keeps requesting
// data for the whole life of the workgroup instead of in bursts between barriers.  DB: a second
// register buffer for the x batches (without it a K part of several batches fetches each batch
// after the previous one has been consumed; the launcher gives such parts the DB form).
constexpr int kShrinkWaves = 4;

// Body of the shrink for one tile.  MASKED: the adapter in the tile's slot has fewer ranks than
// the buffers (eff < R): 16-rank blocks of A[slot] at or above its rank are neither copied to LDS
// nor multiplied, and their partial sums are not written (the expand does not read them).  The
// unmasked instance is the code without any of those tests.
template <typename T, int R, int KR, int XW, bool DB, bool MASKED>
__device__ __forceinline__ void shrink_body(T* __restrict__ s_a, const int32_t* __restrict__ plan, const void* __restrict__ xv,
                                            float* __restrict__ hws, int64_t xs, int sorted_off, int T_, int K, int num_slices, int krange,
                                            int all_slices, const ShrinkSlices& sl, int slice0, int kpart, int slot, int start, int m, int eff) {
  constexpr int RB = (R + 15) / 16;      // 16-rank blocks
  constexpr int NT = kShrinkWaves * kWave;
  constexpr int ASTRIDE = KR + 8;        // padded LDS row: 16 rows x 16 bytes cover all banks once
  constexpr int CPR = KR / 8;            // 16-byte chunks per slab row
  constexpr int TOTAL = R * CPR;         // chunks per slab
  constexpr int CHUNKS = (TOTAL + NT - 1) / NT;  // chunks each thread copies per slab
  constexpr int KS = KR / 32;            // k-steps per slab
  constexpr int XK = XW / 32;            // k-steps per x batch
  constexpr int SPB = XW / KR;           // slabs per x batch
  static_assert(XW % KR == 0 && XK <= 16, "batch shape");

  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int lr = lane & 15, lg = lane >> 4;
  const int nsl = all_slices ? num_slices : 1;
  const int rb_n = MASKED ? (eff + 15) >> 4 : RB;          // 16-rank blocks of A[slot] in use
  const int rows_used = MASKED ? (rb_n * 16 < R ? rb_n * 16 : R) : R;

  const int k0 = kpart * krange;
  const int nbatch = krange / XW;
  const bool active = wave * 16 < m;  // this wavefront's token block exists
  // token row of this lane (lanes past the end of the tile repeat its last token: they feed the
  // MFMA harmlessly and are never written back)
  const int ti = wave * 16 + lr;
  const int row = plan[sorted_off + start + (ti < m ? ti : m - 1)];
  const T* xptr = static_cast<const T*>(xv) + static_cast<int64_t>(row) * xs + k0 + lg * 8;
  const int64_t aoff = static_cast<int64_t>(slot) * R * K + k0;

  i32x4 v[CHUNKS];
  auto request_slab = [&](const T* Aslab) {
#pragma unroll
    for (int i = 0; i < CHUNKS; ++i) {
      const int c = i * NT + tid;
      if constexpr (MASKED) {
        if (i * (NT / CPR) >= rows_used) continue;  // these rows lie beyond the adapter's rank (the same for every thread)
      }
      if (TOTAL % NT == 0 || c < TOTAL) v[i] = load128(Aslab + static_cast<int64_t>(c / CPR) * K + (c % CPR) * 8);
    }
  };
  auto store_slab = [&]() {
#pragma unroll
    for (int i = 0; i < CHUNKS; ++i) {
      const int c = i * NT + tid;
      if constexpr (MASKED) {
        if (i * (NT / CPR) >= rows_used) continue;
      }
      if (TOTAL % NT == 0 || c < TOTAL) *reinterpret_cast<i32x4*>(&s_a[(c / CPR) * ASTRIDE + (c % CPR) * 8]) = v[i];
    }
  };
  auto request_x = [&](Pack8(&buf)[XK], int kc) {
#pragma unroll
    for (int i = 0; i < XK; ++i) buf[i].raw = load128(xptr + kc + i * 32);
  };

  Pack8 xa[XK], xb[DB ? XK : 1];
  f32x4 acc[RB];
  bool first = true;
  // One x batch: `cur` holds it (or is about to), `nxt` receives the following one meanwhile.
  auto run_batch = [&](Pack8(&cur)[XK], Pack8(&nxt)[XK], int si, int b) {
    const T* A = static_cast<const T*>(sl.a[slice0 + si]) + aoff;
    if (DB && active && b + 1 < nbatch) request_x(nxt, (b + 1) * XW);
#pragma unroll
    for (int s = 0; s < SPB; ++s) {
      if (!first) __syncthreads();  // everyone is done reading the previous slab
      first = false;
      store_slab();
      __syncthreads();
      // the slab after this one: same batch, next batch, or the first of the next slice
      if (s + 1 < SPB) request_slab(A + b * XW + (s + 1) * KR);
      else if (b + 1 < nbatch) request_slab(A + (b + 1) * XW);
      else if (si + 1 < nsl) request_slab(static_cast<const T*>(sl.a[slice0 + si + 1]) + aoff);
      if (active) {
#pragma unroll
        for (int i = 0; i < KS; ++i) {
#pragma unroll
          for (int rb = 0; rb < RB; ++rb) {
            if constexpr (MASKED) {
              if (rb >= rb_n) continue;
            }
            const int rr = rb * 16 + lr;
            Pack8 aw;
            aw.raw = *reinterpret_cast<const i32x4*>(&s_a[(rr < R ? rr : R - 1) * ASTRIDE + i * 32 + lg * 8]);
            acc[rb] = Mma<T>::run(aw, cur[s * KS + i], acc[rb]);
          }
        }
      }
    }
    if (!DB && active && b + 1 < nbatch) request_x(cur, (b + 1) * XW);
  };

  request_slab(static_cast<const T*>(sl.a[slice0]) + aoff);
  if (active) request_x(xa, 0);
  for (int si = 0; si < nsl; ++si) {
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) acc[rb] = f32x4{0.f, 0.f, 0.f, 0.f};
    if constexpr (DB) {
      for (int b = 0; b < nbatch; b += 2) {
        run_batch(xa, xb, si, b);
        if (b + 1 < nbatch) run_batch(xb, xa, si, b + 1);
      }
    } else {
      for (int b = 0; b < nbatch; ++b) run_batch(xa, xa, si, b);
    }
    // D layout: lane holds H[rank 16*rb + 4*(lane/16) + i][token lane%16]: four consecutive ranks
    if (active && ti < m) {
      float* dst = hws + ((static_cast<int64_t>(kpart) * T_ + start + ti) * num_slices + slice0 + si) * R;
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const int r0 = rb * 16 + 4 * lg;
        if (r0 < R && (!MASKED || rb < rb_n)) *reinterpret_cast<f32x4*>(dst + r0) = acc[rb];
      }
    }
  }
}


template <typename T, int R, int KR, int XW, bool DB>
__global__ __launch_bounds__(kShrinkWaves* kWave, 2) void sgmv_shrink_kernel(const int32_t* __restrict__ plan, const void* __restrict__ xv,
                                                                             float* __restrict__ hws, int64_t xs, int big_off,
                                                                             int small_off, int big_cap, int sorted_off, int T_, int K,
                                                                             int num_slots, int num_slices, int ksplit, int krange,
                                                                             int all_slices, const int32_t* __restrict__ eff_rank, ShrinkSlices sl) {
  constexpr int ASTRIDE = KR + 8;  // padded LDS row: 16 rows x 16 bytes cover all banks once
  __shared__ __attribute__((aligned(16))) T s_a[R * ASTRIDE];
  // all_slices: the workgroup walks every slice of the projection with the x rows it holds in
  // registers (its K part is a single batch then), instead of one workgroup per slice
  const int slice0 = all_slices ? 0 : blockIdx.y / ksplit, kpart = all_slices ? blockIdx.y : blockIdx.y % ksplit;
  const int tile = blockIdx.z * 8 + blockIdx.x;  // blockIdx.x is the XCD
  const TileRef tr = fetch_tile(plan, big_off, small_off, big_cap, tile, T_, num_slots);
  if (!tr.ok) return;
  // rank of the adapter in this slot (a second, dependent fetch, only with the vector given)
  int eff = R;
  if (R > 16 && eff_rank) {
    eff = eff_rank[tr.slot];
    eff = eff < 0 ? 0 : eff > R ? R : eff;
    if (eff == 0) return;
  }
  if (R > 16 && ((eff + 15) >> 4) < (R + 15) / 16)
    shrink_body<T, R, KR, XW, DB, true>(s_a, plan, xv, hws, xs, sorted_off, T_, K, num_slices, krange, all_slices, sl, slice0, kpart,
                                        tr.slot, tr.start, tr.m, eff);
  else
    shrink_body<T, R, KR, XW, DB, false>(s_a, plan, xv, hws, xs, sorted_off, T_, K, num_slices, krange, all_slices, sl, slice0, kpart,
                                         tr.slot, tr.start, tr.m, eff);
}

// ---- expand -------------------------------------------------------------------------------------
// grid (8, column ranges, tiles / 8), four wavefronts.  OUT[tokens x cols] = H . B[slot]^T with
// the tokens as MFMA rows: in the accumulator layout a lane then holds four tokens of one column,
// and with the B rows of the CPL MFMAs of a span of 16 * CPL columns interleaved (MFMA j takes
// column CPL * (lane % 16) + j) it holds CPL consecutive columns of each of those tokens.
// Sixteen consecutive lanes therefore cover 32 * CPL contiguous bytes of one y row: y is read
// and written in fully coalesced accesses (128-bit for CPL = 8, 64-bit for CPL = 4; the narrower
// span needs half the registers, so more wavefronts and more of their loads are in flight).
// TPF: token blocks whose y rows are requested together.
template <typename T, int N> union alignas(N * sizeof(T)) YVec {
  T e[N];
  uint32_t u[N / 2];
};

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
template <int N> struct YRaw;
template <> struct YRaw<4> { typedef u32x2 type; };
template <> struct YRaw<8> { typedef u32x4 type; };

// y is touched once per launch: with `nt` it is moved with the non-temporal hint so that it does
// not push the B rows, which every tile of a slot re-reads, out of the L2.
template <typename T, int N>
__device__ __forceinline__ YVec<T, N> load_y(const T* p, int nt) {
  typedef typename YRaw<N>::type Raw;
  YVec<T, N> v;
  Raw r = nt ? __builtin_nontemporal_load(reinterpret_cast<const Raw*>(p)) : *reinterpret_cast<const Raw*>(p);
  __builtin_memcpy(&v, &r, sizeof(r));
  return v;
}
template <typename T, int N>
__device__ __forceinline__ void store_y(T* p, const YVec<T, N>& v, int nt) {
  typedef typename YRaw<N>::type Raw;
  Raw r;
  __builtin_memcpy(&r, &v, sizeof(r));
  if (nt) __builtin_nontemporal_store(r, reinterpret_cast<Raw*>(p));
  else *reinterpret_cast<Raw*>(p) = r;
}

// Body of the expand for the tiles of one workgroup.  MASKED: some tile's slot holds an adapter of
// fewer ranks than the buffers: chunks of the intermediate the shrink did not write are not read,
// ranks at or above the adapter's are zero in the intermediate, B columns from that rank on are
// neither fetched nor multiplied.  The unmasked instance is the code without any of those tests.
template <typename T, int R, int CPL, int TPF, int G, bool MASKED>
__device__ __forceinline__ void expand_body(T* __restrict__ s_h, int* __restrict__ s_row, int* __restrict__ s_slot, int* __restrict__ s_m,
                                            int* __restrict__ s_eff, const int32_t* __restrict__ plan, const float* __restrict__ hws,
                                            void* __restrict__ yv_, int64_t ys, int sorted_off, int T_, int num_slices, int ksplit,
                                            float scaling, int nt, const ExpandSplit& sp, const int (&slot)[G], const int (&start)[G],
                                            const int (&m)[G], const int (&eff)[G]) {
  constexpr int TB = MLORA_TILE_BIG / 16;
  constexpr int NB = TB / TPF;           // y batches per tile
  constexpr int STEPS = G * NB;          // (tile, batch) steps of a span
  constexpr int KSTEPS = (R + 31) / 32;  // MFMA k-steps
  constexpr int HSTRIDE = 2 * R + 8;     // padded LDS row: R leading parts, R remainders
  constexpr int NT = kExpandWaves * kWave;
  constexpr int CPR = R / 8;             // groups of eight ranks per token
  constexpr int SPAN = 16 * CPL;         // columns of one span
  constexpr int HC = (MLORA_TILE_BIG * CPR + NT - 1) / NT;  // H chunks per thread and tile

  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int lr = lane & 15, lg = lane >> 4;

  // token rows -> LDS (entries past the end of a tile repeat its last token: a valid row to read,
  // never written)
#pragma unroll
  for (int g = 0; g < G; ++g) {
    if (tid == 0) { s_slot[g] = slot[g]; s_m[g] = m[g]; s_eff[g] = eff[g]; }
    if (m[g] > 0 && tid < MLORA_TILE_BIG) s_row[g * MLORA_TILE_BIG + tid] = plan[sorted_off + start[g] + (tid < m[g] ? tid : m[g] - 1)];
  }
  __syncthreads();

  // A wavefront's work is a sequence of items: for each of its spans of 16 * CPL columns, the
  // (tile, y batch) steps that hold tokens.  The y rows of the item after the current one are
  // always in flight, and those of the first item (and its B rows) go out before the H tiles
  // are staged, so that the stream of y never waits for anything but itself.
  T* const ybase = static_cast<T*>(yv_) + sp.y_col;
  auto next_step = [&](int st) {
    for (++st; st < STEPS; ++st)
      if (s_m[st / NB] > (st % NB) * TPF * 16) break;
    return st;
  };
  const int first_step = next_step(-1);  // exists: some tile holds tokens
  auto column = [&](int c0) {  // first of this lane's CPL columns, clamped into the range
    const int c = c0 + CPL * lr;
    return c < sp.n1 ? c : sp.n1 - 8;
  };
  auto issue_y = [&](YVec<T, CPL>(&buf)[TPF][4], int c0, int st) {
    const int g = st / NB, tp = (st % NB) * TPF, cl = column(c0);
#pragma unroll
    for (int u = 0; u < TPF; ++u) {
      const i32x4 rows = *reinterpret_cast<const i32x4*>(&s_row[g * MLORA_TILE_BIG + (tp + u) * 16 + 4 * lg]);
#pragma unroll
      for (int i = 0; i < 4; ++i) buf[u][i] = load_y<T, CPL>(ybase + static_cast<int64_t>(rows[i]) * ys + cl, nt);
    }
  };
  Pack8 bop[CPL][KSTEPS];
  int b_slot = -1, b_c0 = -1;  // what bop holds
  int b_ks = KSTEPS;  // k-steps of the slot bop holds
  auto load_b = [&](int c0, int sg, int eg) {
    // the B rows of the span (lanes whose chunk lies beyond the rank fetch a valid chunk anyway,
    // their H operand is zero; columns past the range repeat the last one and are never stored)
    const T* B = static_cast<const T*>(sp.b) + static_cast<int64_t>(sg) * sp.n * R;
    if (!MASKED || eg >= R) {
#pragma unroll
      for (int j = 0; j < CPL; ++j) {
        int n = c0 + CPL * lr + j;
        n = n < sp.n1 ? n : sp.n1 - 1;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
          const int kc = (lg + 4 * ks) & (R / 8 - 1);
          bop[j][ks].raw = load128(B + static_cast<int64_t>(n) * R + kc * 8);
        }
      }
    } else if constexpr (MASKED) {
      // an adapter of lower rank: only its own chunks of eight ranks are fetched, the rest of the
      // operand is zero, and what the boundary chunk holds beyond the rank is masked out
      const int eg8 = (eg + 7) >> 3;
#pragma unroll
      for (int j = 0; j < CPL; ++j) {
        int n = c0 + CPL * lr + j;
        n = n < sp.n1 ? n : sp.n1 - 1;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
          const int kc = lg + 4 * ks;
          if (kc < eg8) {
            bop[j][ks].raw = load128(B + static_cast<int64_t>(n) * R + kc * 8);
            if (eg & 7) mask_ranks(bop[j][ks], kc * 8, eg);
          } else {
            bop[j][ks].raw = i32x4{0, 0, 0, 0};
          }
        }
      }
    }
    b_slot = sg;
    b_c0 = c0;
    if constexpr (MASKED) b_ks = (eg + 31) >> 5;
  };
  auto process = [&](YVec<T, CPL>(&buf)[TPF][4], int c0, int st) {
    const int g = st / NB, tp = (st % NB) * TPF;
    const int mg = s_m[g], sg = s_slot[g];
    if (sg != b_slot || c0 != b_c0) load_b(c0, sg, s_eff[g]);
    const T* hg = s_h + g * MLORA_TILE_BIG * HSTRIDE;
    const int c = c0 + CPL * lr;
    const bool col_ok = c < sp.n1;
#pragma unroll
    for (int u = 0; u < TPF; ++u) {
      const int tb = tp + u;
      if (tb * 16 >= mg) continue;
      Pack8 hop[KSTEPS], hlo[KSTEPS];
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        const int kc = lg + 4 * ks;
        if (kc * 8 < R) {
          hop[ks].raw = *reinterpret_cast<const i32x4*>(&hg[(tb * 16 + lr) * HSTRIDE + kc * 8]);
          hlo[ks].raw = *reinterpret_cast<const i32x4*>(&hg[(tb * 16 + lr) * HSTRIDE + R + kc * 8]);
        } else {
          hop[ks].raw = i32x4{0, 0, 0, 0};
          hlo[ks].raw = i32x4{0, 0, 0, 0};
        }
      }
      f32x4 out[CPL];
#pragma unroll
      for (int j = 0; j < CPL; ++j) {
        out[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
          if constexpr (MASKED && KSTEPS > 1) {
            if (ks >= b_ks) continue;
          }
          out[j] = Mma<T>::run(hlo[ks], bop[j][ks], out[j]);
          out[j] = Mma<T>::run(hop[ks], bop[j][ks], out[j]);
        }
      }
      // lane holds out[token 16*tb + 4*lg + i][column c0 + CPL*lr + j]
      const i32x4 rows = *reinterpret_cast<const i32x4*>(&s_row[g * MLORA_TILE_BIG + tb * 16 + 4 * lg]);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (col_ok && tb * 16 + 4 * lg + i < mg) {
          YVec<T, CPL> r;
#pragma unroll
          for (int j = 0; j < CPL; ++j) r.e[j] = from_f32<T>(to_f32(buf[u][i].e[j]) + out[j][i]);
          store_y<T, CPL>(ybase + static_cast<int64_t>(rows[i]) * ys + c, r, nt);
        }
      }
    }
  };

  YVec<T, CPL> ya[TPF][4], yb[TPF][4];
  int c0 = sp.n0 + wave * SPAN, st = first_step;
  const bool has_work = c0 < sp.n1;
  if (has_work) {
    load_b(c0, s_slot[st / NB], s_eff[st / NB]);
    issue_y(ya, c0, st);
  }

  // H tiles -> LDS: K partials summed (always in the same order), scaled, split into leading
  // part and remainder; absent tokens get zeros.  All loads of a tile are in flight together.
  {
    const int64_t hrow = static_cast<int64_t>(num_slices) * R;
    const int64_t part = static_cast<int64_t>(T_) * hrow;
#pragma unroll
    for (int g = 0; g < G; ++g) {
      if (m[g] == 0) continue;
      const float* src = hws + static_cast<int64_t>(start[g]) * hrow + sp.slice * R;
      f32x4 t[HC][kMaxKSplit][2];
#pragma unroll
      for (int h = 0; h < HC; ++h) {
        const int c = h * NT + tid;
        int tok = c / CPR;
        tok = tok < m[g] ? tok : m[g] - 1;
        const float* q = src + tok * hrow + (c % CPR) * 8;
        const bool used = !MASKED || (c % CPR) * 8 < ((eff[g] + 15) & ~15);  // the shrink wrote this chunk
#pragma unroll
        for (int kp = 0; kp < kMaxKSplit; ++kp) {
          if (kp < ksplit) {
            if (used) {
              t[h][kp][0] = *reinterpret_cast<const f32x4*>(q + kp * part);
              t[h][kp][1] = *reinterpret_cast<const f32x4*>(q + kp * part + 4);
            } else {
              t[h][kp][0] = f32x4{0.f, 0.f, 0.f, 0.f};
              t[h][kp][1] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
          }
        }
      }
#pragma unroll
      for (int h = 0; h < HC; ++h) {
        const int c = h * NT + tid, tok = c / CPR, ch = c % CPR;
        if ((MLORA_TILE_BIG * CPR) % NT != 0 && c >= MLORA_TILE_BIG * CPR) continue;
        f32x4 s0 = t[h][0][0], s1 = t[h][0][1];
#pragma unroll
        for (int kp = 1; kp < kMaxKSplit; ++kp) {
          if (kp < ksplit) {
            s0[0] += t[h][kp][0][0]; s0[1] += t[h][kp][0][1]; s0[2] += t[h][kp][0][2]; s0[3] += t[h][kp][0][3];
            s1[0] += t[h][kp][1][0]; s1[1] += t[h][kp][1][1]; s1[2] += t[h][kp][1][2]; s1[3] += t[h][kp][1][3];
          }
        }
        Pack8 hi, lo;
        float v[8], back[8], rem[8];
        const float live = tok < m[g] ? scaling : 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          v[i] = (!MASKED || ch * 8 + i < eff[g]) ? s0[i] * live : 0.f;  // ranks the adapter does not have contribute nothing
          v[4 + i] = (!MASKED || ch * 8 + 4 + i < eff[g]) ? s1[i] * live : 0.f;
        }
        pack8<T>(v, hi);
        unpack8<T>(hi, back);
#pragma unroll
        for (int i = 0; i < 8; ++i) rem[i] = v[i] - back[i];
        pack8<T>(rem, lo);
        *reinterpret_cast<i32x4*>(&s_h[(g * MLORA_TILE_BIG + tok) * HSTRIDE + ch * 8]) = hi.raw;
        *reinterpret_cast<i32x4*>(&s_h[(g * MLORA_TILE_BIG + tok) * HSTRIDE + R + ch * 8]) = lo.raw;
      }
    }
  }
  __syncthreads();
  if (!has_work) return;

  // two y buffers, used in turn
  auto advance = [&](int& nc0, int& nst) {  // item after (c0, st); false when there is none
    nst = next_step(st);
    nc0 = c0;
    if (nst >= STEPS) {
      nst = first_step;
      nc0 = c0 + kExpandWaves * SPAN;
    }
    return nc0 < sp.n1;
  };
  for (;;) {
    int nc0, nst;
    bool more = advance(nc0, nst);
    if (more) issue_y(yb, nc0, nst);
    process(ya, c0, st);
    if (!more) break;
    c0 = nc0;
    st = nst;
    more = advance(nc0, nst);
    if (more) issue_y(ya, nc0, nst);
    process(yb, c0, st);
    if (!more) break;
    c0 = nc0;
    st = nst;
  }
}

template <typename T, int R, int CPL, int TPF, int G>
__global__ __launch_bounds__(kExpandWaves* kWave, 2) void sgmv_expand_kernel(const int32_t* __restrict__ plan, const float* __restrict__ hws,
                                                                             void* __restrict__ yv_, int64_t ys, int big_off, int small_off,
                                                                             int big_units, int sorted_off, int T_, int num_slots,
                                                                             int num_slices, int ksplit, float scaling, int nt,
                                                                             const int32_t* __restrict__ eff_rank, ExpandSplits splits) {
  constexpr int HSTRIDE = 2 * R + 8;     // padded LDS row: R leading parts, R remainders
  __shared__ __attribute__((aligned(16))) T s_h[G * MLORA_TILE_BIG * HSTRIDE];
  __shared__ __attribute__((aligned(16))) int s_row[G * MLORA_TILE_BIG];
  __shared__ int s_slot[G], s_m[G], s_eff[G];

  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int lr = lane & 15, lg = lane >> 4;
  // A workgroup takes G consecutive 64-token tiles (consecutive tiles mostly belong to one slot,
  // whose B rows then stay in registers across them), or, past `big_units`, one short segment.
  const int unit = blockIdx.z * 8 + blockIdx.x;  // blockIdx.x is the XCD
  const bool is_big = unit < big_units;
  const int sidx = is_big ? 0 : unit - big_units;

  // header and every candidate record are requested together (all addresses are in bounds for
  // the whole grid)
  const i32x4 hdr0 = *reinterpret_cast<const i32x4*>(plan);
  const i32x4 hdr1 = *reinterpret_cast<const i32x4*>(plan + 4);
  const i32x4 hdr2 = *reinterpret_cast<const i32x4*>(plan + 8);
  const i32x4 small = *reinterpret_cast<const i32x4*>(plan + small_off + sidx * MLORA_SMALL_TILE_WORDS);
  i32x4 big[G];
#pragma unroll
  for (int g = 0; g < G; ++g) big[g] = reinterpret_cast<const i32x4*>(plan + big_off)[is_big ? unit * G + g : 0];
  const ExpandSplit sp = splits.split[blockIdx.y];
  const int n_big = hdr2[MLORA_PLAN_TILES_LONG_BIG - 8], n_short = hdr1[MLORA_PLAN_TILES_SHORT - 4];
  int slot[G], start[G], m[G], any = 0;
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const bool have = is_big ? unit * G + g < n_big : (g == 0 && sidx < n_short);
    slot[g] = is_big ? big[g][0] : small[0];
    start[g] = is_big ? big[g][1] : small[2];
    m[g] = is_big ? big[g][2] : small[1];
    if (!have || m[g] <= 0 || slot[g] < 0 || slot[g] >= num_slots) m[g] = 0;
  }
  // rank of the adapter in each tile's slot (a second, dependent fetch, only with the vector
  // given): ranks at or above it are left out of the intermediate, of the B rows and of the MFMAs
  int eff[G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    eff[g] = R;
    if (eff_rank && m[g] > 0) {
      const int e = eff_rank[slot[g]];
      eff[g] = e < 0 ? 0 : e > R ? R : e;
      if (eff[g] == 0) m[g] = 0;  // nothing resident: the tile is skipped
    }
    any |= m[g];
  }
  const int usable = int(hdr0[MLORA_PLAN_MAGIC] == MLORA_PLAN_MAGIC_VALUE) & int(hdr0[MLORA_PLAN_NUM_TOKENS] == T_) &
                     int(hdr0[MLORA_PLAN_MAX_SLOTS] == num_slots) & int(any > 0) & int(sp.n0 < sp.n1);
  if (!usable) return;

  bool masked = false;
#pragma unroll
  for (int g = 0; g < G; ++g) masked |= m[g] > 0 && eff[g] < R;
  if (masked)
    expand_body<T, R, CPL, TPF, G, true>(s_h, s_row, s_slot, s_m, s_eff, plan, hws, yv_, ys, sorted_off, T_, num_slices, ksplit, scaling, nt,
                                         sp, slot, start, m, eff);
  else
    expand_body<T, R, CPL, TPF, G, false>(s_h, s_row, s_slot, s_m, s_eff, plan, hws, yv_, ys, sorted_off, T_, num_slices, ksplit, scaling, nt,
                                          sp, slot, start, m, eff);
}

// The fp32 partials of the intermediate live behind the head of the workspace.
float* partials_of(const MloraAddArgs* a) { return reinterpret_cast<float*>(static_cast<char*>(a->workspace) + MLORA_WORKSPACE_HEAD_BYTES); }
size_t partials_room(const MloraAddArgs* a) {
  return a->workspace_bytes > MLORA_WORKSPACE_HEAD_BYTES ? static_cast<size_t>(a->workspace_bytes) - MLORA_WORKSPACE_HEAD_BYTES : 0;
}

// Diagnostic knobs, read from the environment once and again after mlora_reload_knobs().
struct SgmvKnobs {
  int generation = -1, nt_hint, kr, ksplit, all_slices, xdb, group, wgs, nt, cpl;
  void read() {
    generation = knob_generation();
    nt_hint = env_int("MLORA_SGMV_NT_HINT", 0);
    kr = env_int("MLORA_SGMV_KR", 0);
    ksplit = env_int("MLORA_SGMV_KSPLIT", 0);
    all_slices = env_int("MLORA_SGMV_ALL_SLICES", 3);
    xdb = env_int("MLORA_SGMV_XDB", 1);
    group = env_int("MLORA_SGMV_GROUP", 0);
    wgs = env_int("MLORA_SGMV_WGS", 2048);
    nt = env_int("MLORA_SGMV_NT", 0);
    cpl = env_int("MLORA_SGMV_CPL", 8);
  }
};
const SgmvKnobs& sgmv_knobs() {
  static SgmvKnobs k;
  if (k.generation != knob_generation()) k.read();
  return k;
}

struct ShrinkLaunch {
  const MloraAddArgs* a;
  PlanLayout lay;
  ShrinkSlices sl;
  int tiles8;   // grid extent over tiles / 8
  int big_cap;  // workgroups below this index take 64-token tiles, the rest short segments
  int ksplit, krange, all_slices;
};

template <typename T, int R, int KR, int XW, bool DB>
void launch_shrink_one(const ShrinkLaunch& l) {
  const MloraAddArgs* a = l.a;
  dim3 grid(8, static_cast<unsigned>(l.all_slices ? l.ksplit : a->num_slices * l.ksplit), static_cast<unsigned>(l.tiles8));
  hipLaunchKernelGGL((sgmv_shrink_kernel<T, R, KR, XW, DB>), grid, dim3(kShrinkWaves * kWave), 0, static_cast<hipStream_t>(a->stream),
                     a->plan, a->x, partials_of(a), a->x_stride, l.lay.big_off, l.lay.small_off, l.big_cap,
                     l.lay.sorted_off, a->num_tokens, a->k, a->num_slots, a->num_slices, l.ksplit, l.krange, l.all_slices, a->effective_rank, l.sl);
}

// (slab width, x batch width): 128/128 and 256/256 with two x buffers, 256/512 and 512/512 with one
template <typename T, int R>
void launch_shrink_slab(const ShrinkLaunch& l, int kr, int xw) {
  if (kr == 128) launch_shrink_one<T, R, 128, 128, true>(l);
  else if (kr == 256 && xw == 256) launch_shrink_one<T, R, 256, 256, true>(l);
  else if (kr == 256) launch_shrink_one<T, R, 256, 512, false>(l);
  else launch_shrink_one<T, R, 512, 512, false>(l);
}

template <typename T>
void launch_shrink_rank(const ShrinkLaunch& l, int kr, int xw) {
  switch (l.a->r) {
    case 8: launch_shrink_slab<T, 8>(l, kr, xw); break;
    case 16: launch_shrink_slab<T, 16>(l, kr, xw); break;
    case 32: launch_shrink_slab<T, 32>(l, kr, xw); break;
    default: launch_shrink_slab<T, 64>(l, kr, xw); break;
  }
}

template <typename T, int R>
void launch_expand_group(const MloraAddArgs* a, const PlanLayout& lay, int big_units, dim3 grid, int ksplit, int cpl, int group,
                         const ExpandSplits& sp) {
  hipStream_t st = static_cast<hipStream_t>(a->stream);
  const float* h = partials_of(a);
  const int nt = sgmv_knobs().nt_hint;
#define MLORA_EXPAND(CPL_, TPF_, G_)                                                                                       \
  hipLaunchKernelGGL((sgmv_expand_kernel<T, R, CPL_, TPF_, G_>), grid, dim3(kExpandWaves* kWave), 0, st, a->plan, h, a->y, \
                     a->y_stride, lay.big_off, lay.small_off, big_units, lay.sorted_off, a->num_tokens, a->num_slots,      \
                     a->num_slices, ksplit, a->scaling, nt, a->effective_rank, sp)
  if (cpl == 4) {
    if (group == 4) MLORA_EXPAND(4, 4, 4); else if (group == 2) MLORA_EXPAND(4, 4, 2); else MLORA_EXPAND(4, 4, 1);
  } else {
    if (group == 4) MLORA_EXPAND(8, 2, 4); else if (group == 2) MLORA_EXPAND(8, 2, 2); else MLORA_EXPAND(8, 2, 1);
  }
#undef MLORA_EXPAND
}

template <typename T>
void launch_expand_rank(const MloraAddArgs* a, const PlanLayout& lay, int big_units, dim3 grid, int ksplit, int cpl, int group,
                        const ExpandSplits& sp) {
  switch (a->r) {
    case 8: launch_expand_group<T, 8>(a, lay, big_units, grid, ksplit, cpl, group, sp); break;
    case 16: launch_expand_group<T, 16>(a, lay, big_units, grid, ksplit, cpl, group, sp); break;
    case 32: launch_expand_group<T, 32>(a, lay, big_units, grid, ksplit, cpl, group, sp); break;
    default: launch_expand_group<T, 64>(a, lay, big_units, grid, ksplit, cpl, group, sp); break;
  }
}

// Column ranges of about `nt` columns (a multiple of 512: four wavefronts of 128 columns).
int fill_splits(const MloraAddArgs* a, int nt, ExpandSplit* out) {
  nt = (nt + 511) & ~511;
  if (nt < 512) nt = 512;
  int total;
  for (;;) {
    total = 0;
    for (int i = 0; i < a->num_slices; ++i) total += (a->slices[i].n + nt - 1) / nt;
    if (total <= kMaxSplits) break;
    nt *= 2;
  }
  int s = 0;
  for (int i = 0; i < a->num_slices; ++i) {
    const MloraSlice& sl = a->slices[i];
    for (int n0 = 0; n0 < sl.n; n0 += nt) {
      ExpandSplit& sp = out[s++];
      sp.b = sl.b; sp.n = sl.n; sp.y_col = sl.y_col; sp.slice = i; sp.pad = 0;
      sp.n0 = n0; sp.n1 = n0 + nt < sl.n ? n0 + nt : sl.n;
    }
  }
  return total;
}

}  // namespace

// One fp32 partial of the intermediate: [T, slices, r].
static size_t partial_bytes(int num_tokens, int num_slices, int r) {
  return static_cast<size_t>(num_tokens) * static_cast<size_t>(num_slices) * static_cast<size_t>(r) * sizeof(float);
}

size_t sgmv_workspace_bytes(int num_tokens, int num_slices, int r, int dtype) {
  (void)dtype;
  if (num_tokens <= 0 || num_slices <= 0 || r <= 0) return 0;
  return MLORA_WORKSPACE_HEAD_BYTES + kMaxKSplit * partial_bytes(num_tokens, num_slices, r);
}

bool sgmv_supported(const MloraAddArgs* a) { return a->k % 128 == 0 && a->k >= 128; }

// A workspace that holds at least one partial can be used (fewer K parts are taken then).
bool sgmv_workspace_ok(const MloraAddArgs* a) {
  if (!a->workspace || (reinterpret_cast<uintptr_t>(a->workspace) & 255)) return false;
  for (int i = 0; i < a->num_slices; ++i)
    if (a->slices[i].n <= 0) return false;  // every slice owns a workspace column block
  return partials_room(a) >= partial_bytes(a->num_tokens, a->num_slices, a->r);
}

// Every segment of the batch: 64-token tiles of the long ones, one short tile each for the rest.
int launch_sgmv(const MloraAddArgs* a) {
  ShrinkLaunch l;
  l.a = a;
  l.lay = plan_layout(a->num_tokens, a->num_slots);
  l.big_cap = (l.lay.cap_big + 7) & ~7;
  int short_cap = a->num_slots < a->num_tokens ? a->num_slots : a->num_tokens;  // a short segment is one small tile
  if (short_cap > l.lay.cap_small) short_cap = l.lay.cap_small;
  const int cap = l.big_cap + ((short_cap + 7) & ~7);
  if (cap == 0) return 0;
  l.tiles8 = cap / 8;
  int cols = 0;
  for (int i = 0; i < a->num_slices; ++i) {
    cols += a->slices[i].n;
    l.sl.a[i] = a->slices[i].a;
  }
  for (int i = a->num_slices; i < MLORA_MAX_SLICES; ++i) l.sl.a[i] = nullptr;
  if (cols == 0) return 0;
  const int est_tiles = a->num_tokens / MLORA_TILE_BIG + 1;

  // shrink: x batch width (what a wavefront holds in registers: 512 columns when K allows), A
  // slab width (a whole batch: on the prefill and the mixed batch 128-, 256- and 512-column
  // slabs measured within 2 % of each other), then K parts so that the grid has a few
  // workgroups per compute unit
  int xw = 512;
  while (xw > 128 && a->k % xw != 0) xw /= 2;
  int kr = sgmv_knobs().kr;
  if (kr != 128 && kr != 256 && kr != 512) kr = xw;
  if (kr > xw) kr = xw;
  if (kr == 128) xw = 128;  // 128-column slabs come with 128-column batches only
  const int max_parts = static_cast<int>(partials_room(a) / partial_bytes(a->num_tokens, a->num_slices, a->r));
  int ksplit = sgmv_knobs().ksplit;
  if (ksplit <= 0) {
    ksplit = 1;
    while (ksplit < kMaxKSplit && static_cast<long long>(est_tiles) * a->num_slices * ksplit < 512 && a->k % (xw * ksplit * 2) == 0) ksplit *= 2;
  }
  if (ksplit > max_parts) ksplit = max_parts;
  if (ksplit > kMaxKSplit) ksplit = kMaxKSplit;
  while (ksplit > 1 && a->k % (xw * ksplit) != 0) --ksplit;
  // three or more slices: one workgroup walks them all with the x rows it already holds, when
  // its K part is a single batch (measured on the prefill batch: qkv 31.9 -> 29.6 us per call;
  // with two slices the shorter chain of separate workgroups wins, gate_up 76.6 vs 77.8)
  l.all_slices = 0;
  if (a->num_slices >= sgmv_knobs().all_slices) {
    const int parts = a->k / xw;
    if (parts <= kMaxKSplit && parts <= max_parts) {
      ksplit = parts;
      l.all_slices = 1;
    }
  }
  l.ksplit = ksplit;
  l.krange = a->k / ksplit;
  // a K part of several batches: the form with two x buffers (256-column batches)
  if (xw == 512 && l.krange > xw && sgmv_knobs().xdb) { xw = 256; kr = 256; }
  if (a->dtype == MLORA_DTYPE_BF16) launch_shrink_rank<__bf16>(l, kr, xw);
  else launch_shrink_rank<_Float16>(l, kr, xw);
  int rc = check_launch("mlora_add_lora(sgmv shrink)");
  if (rc) return rc;

  // expand: consecutive tiles per workgroup (they share their B rows when they share their
  // slot), then column ranges so that the grid has about 2048 workgroups
  ExpandSplits splits;
  int group = sgmv_knobs().group;
  if (group != 1 && group != 2 && group != 4) group = (cols >= 4096 && est_tiles >= 64) ? 4 : 1;  // wide projections only: narrow ones need the workgroups
  const int target = sgmv_knobs().wgs;
  int nt = sgmv_knobs().nt;
  if (nt <= 0) {
    const long long want = static_cast<long long>(cols) * (est_tiles / group + 1) / (target > 0 ? target : 1);
    nt = want > 8192 ? 8192 : static_cast<int>(want);
  }
  const int nsplit = fill_splits(a, nt, splits.split);
  const int cpl = sgmv_knobs().cpl == 4 ? 4 : 8;
  const int big_units = l.big_cap / group;  // big_cap is a multiple of 32: a multiple of 8 again
  const int units = big_units + (l.tiles8 * 8 - l.big_cap);
  dim3 grid(8, static_cast<unsigned>(nsplit), static_cast<unsigned>(units / 8));
  if (a->dtype == MLORA_DTYPE_BF16) launch_expand_rank<__bf16>(a, l.lay, big_units, grid, ksplit, cpl, group, splits);
  else launch_expand_rank<_Float16>(a, l.lay, big_units, grid, ksplit, cpl, group, splits);
  return check_launch("mlora_add_lora(sgmv expand)");
}

}  // namespace mlora
