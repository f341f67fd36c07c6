// Shared by the two-launch and the one-launch form of the long-segment kernels: tile lookup, the
// shrink of one (tile, slices, K part) and the expand of one (group of tiles, column range) as
// device functions, and the host-side helpers both launchers use.
#pragma once
#include <type_traits>

#include "common.h"
#include "launch.h"

namespace mlora {

namespace {

MLORA_TRACE_DECL

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
  int plan_ok;  // the plan's header is that of this call's batch shape
};

// Position in the tile lists of workgroup (x, ., z) of a grid (8, ., big_cap / 8 + short segments / 8):
// the first big_cap / 8 layers take the 64-token tiles, XCD x its own block of the list; the layers
// behind them take the short segments, eight abreast.  Positions from big_cap on are short segments.
__device__ __forceinline__ int tile_position(int big_cap) {
  const int blk = big_cap >> 3, z = blockIdx.z, x = blockIdx.x;
  return z < blk ? x * blk + z : big_cap + (z - blk) * 8 + x;
}

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
  // the position holds a tile of this plan: places of the list of 64-token tiles that hold none carry count 0
  const bool present = is_big ? true : sidx < hdr1[MLORA_PLAN_TILES_SHORT - 4];
  t.ok = int(hdr0[MLORA_PLAN_MAGIC] == MLORA_PLAN_MAGIC_VALUE) & int(hdr0[MLORA_PLAN_NUM_TOKENS] == T_) &
         int(hdr0[MLORA_PLAN_MAX_SLOTS] == num_slots) & int(present) & int(t.m > 0) & int(t.slot >= 0) &
         int(t.slot < num_slots);
  t.plan_ok = int(hdr0[MLORA_PLAN_MAGIC] == MLORA_PLAN_MAGIC_VALUE) & int(hdr0[MLORA_PLAN_NUM_TOKENS] == T_) &
              int(hdr0[MLORA_PLAN_MAX_SLOTS] == num_slots);
  return t;
}

// Token row at position `ti` of tile `tile`.  Where it lies follows from the tile's number alone (a
// 64-token tile has its row list behind the big-tile records, a short segment carries its rows in
// its record), so it is requested together with the record instead of after it.  Positions past
// the tile's count hold a valid row as well (a tile's own in a short segment's record, row 0 in a
// big tile's list): read, never written.
__device__ __forceinline__ int tile_row(const int32_t* __restrict__ plan, int bigrows_off, int small_off, int big_cap, int tile, int ti) {
  const bool is_big = tile < big_cap;
  const int at = is_big ? bigrows_off + tile * MLORA_TILE_BIG + ti
                        : small_off + (tile - big_cap) * MLORA_SMALL_TILE_WORDS + MLORA_SMALL_TILE_ROWS + (ti & (MLORA_TILE_SMALL - 1));
  return plan[at];
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
//
// SC1: the partial sums leave with agent-scope stores (they pass the compute unit's and the XCD's
// caches on their way), for readers in other workgroups of the same launch.
//
// TO_LDS: the workgroup multiplies the whole of K for one slice and expands the result itself: the
// sums do not leave the compute unit but go to LDS (`s_h`, which may be the memory of `s_a`) as the
// expand wants its operand: scaled, split into a leading part and a remainder of operand precision,
// zeros for positions past the tile's count and for ranks the adapter does not have.
template <typename T, int R, int KR, int XW, bool DB, bool MASKED, bool SC1 = false, bool TO_LDS = false>
__device__ __forceinline__ void shrink_body(T* __restrict__ s_a, const void* __restrict__ xv, float* __restrict__ hws, int64_t xs, int T_, int K,
                                            int num_slices, int krange, int all_slices, const ShrinkSlices& sl, int slice0, int kpart, int slot,
                                            int start, int m, int eff, int row, T* s_h = nullptr, float scaling = 1.f) {
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
  // `row`: token row of this lane, position wave * 16 + lane % 16 of the tile (positions past the
  // end of the tile name valid rows too: they feed the MFMA harmlessly and are never
  // written back)
  const int ti = wave * 16 + lr;
  MLORA_STAMP(2);  // shrink: body entered (the token rows were requested with the record)
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

  // D layout: lane holds H[rank 16*rb + 4*(lane/16) + i][token lane%16]: four consecutive ranks
  auto write_partials = [&](const f32x4(&part)[RB], int si) {
    if constexpr (TO_LDS) {
      constexpr int HSTRIDE = 2 * R + 8;  // the expand's row: R leading parts, R remainders
      typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
      __syncthreads();  // every wavefront is done with the last slab: its memory may be the intermediate's
      const float live = (active && ti < m) ? scaling : 0.f;
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const int r0 = rb * 16 + 4 * lg;
        if (r0 < R) {
          T hi[4], lo[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float v = r0 + i < eff ? part[rb][i] * live : 0.f;  // (eff = R unless the adapter has fewer ranks)
            hi[i] = from_f32<T>(v);
            lo[i] = from_f32<T>(v - to_f32(hi[i]));
          }
          u32x2_t h2, l2;
          __builtin_memcpy(&h2, hi, 8);
          __builtin_memcpy(&l2, lo, 8);
          *reinterpret_cast<u32x2_t*>(&s_h[ti * HSTRIDE + r0]) = h2;
          *reinterpret_cast<u32x2_t*>(&s_h[ti * HSTRIDE + R + r0]) = l2;
        }
      }
      return;
    }
    if (active && ti < m) {
      float* dst = hws + ((static_cast<int64_t>(kpart) * T_ + start + ti) * num_slices + slice0 + si) * R;
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const int r0 = rb * 16 + 4 * lg;
        if (r0 < R && (!MASKED || rb < rb_n)) {
          if constexpr (SC1) {
            uint64_t* q = reinterpret_cast<uint64_t*>(dst + r0);
            __hip_atomic_store(q, (static_cast<uint64_t>(__float_as_uint(part[rb][1])) << 32) | __float_as_uint(part[rb][0]), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(q + 1, (static_cast<uint64_t>(__float_as_uint(part[rb][3])) << 32) | __float_as_uint(part[rb][2]), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
          } else {
            *reinterpret_cast<f32x4*>(dst + r0) = part[rb];
          }
        }
      }
    }
  };

  if constexpr (!DB && KR == XW && KR >= 256) {
    // A batch that is one slab: slab and batch are requested in NS column pieces, piece after
    // piece (A piece, then the x columns it meets), all of them up front; a piece is copied to LDS
    // and multiplied as soon as it is there, while the later ones are still on their way.  A piece
    // of the slab has its own place in LDS and NS - 1 barriers lie between two uses of a place, so
    // one barrier per piece is enough; a piece's registers take the next slab's piece (next batch
    // or next slice) as soon as they are stored.
    constexpr int NS = MASKED ? 2 : 4, SW = KR / NS, SCPR = SW / 8, STOTAL = R * SCPR, SCH = (STOTAL + NT - 1) / NT, KSS = KS / NS;
    static_assert(KS % NS == 0, "pieces of whole k-steps");
    i32x4 v[NS][SCH];
    Pack8 xa[XK];
    f32x4 acc[RB];
    auto request_piece = [&](const T* Aslab, int s, i32x4(&buf)[SCH]) {
#pragma unroll
      for (int i = 0; i < SCH; ++i) {
        const int c = i * NT + tid;
        if constexpr (MASKED) {
          if (i * (NT / SCPR) >= rows_used) continue;  // rows beyond the adapter's rank (the same for every thread)
        }
        if (STOTAL % NT == 0 || c < STOTAL) buf[i] = load128(Aslab + static_cast<int64_t>(c / SCPR) * K + s * SW + (c % SCPR) * 8);
      }
    };
    auto store_piece = [&](int s, const i32x4(&buf)[SCH]) {
#pragma unroll
      for (int i = 0; i < SCH; ++i) {
        const int c = i * NT + tid;
        if constexpr (MASKED) {
          if (i * (NT / SCPR) >= rows_used) continue;
        }
        if (STOTAL % NT == 0 || c < STOTAL) *reinterpret_cast<i32x4*>(&s_a[(c / SCPR) * ASTRIDE + s * SW + (c % SCPR) * 8]) = buf[i];
      }
    };
    auto request_x_piece = [&](int kc, int s) {
#pragma unroll
      for (int i = 0; i < KSS; ++i) xa[s * KSS + i].raw = load128(xptr + kc + (s * KSS + i) * 32);
    };
    {
      const T* A0 = static_cast<const T*>(sl.a[slice0]) + aoff;
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        // (piece by piece: with every A piece ahead of the x columns the prefill step takes 3816
        // against 3753 us)
        request_piece(A0, s, v[s]);
        if (active) request_x_piece(0, s);
      }
    }
    MLORA_STAMP(3);  // shrink: first slab and first x batch requested (the token rows are here)
    for (int si = 0; si < nsl; ++si) {
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) acc[rb] = f32x4{0.f, 0.f, 0.f, 0.f};
      for (int b = 0; b < nbatch; ++b) {
        // the slab after this one: next batch, or the first of the next slice
        const T* An = nullptr;
        if (b + 1 < nbatch) An = static_cast<const T*>(sl.a[slice0 + si]) + aoff + (b + 1) * XW;
        else if (si + 1 < nsl) An = static_cast<const T*>(sl.a[slice0 + si + 1]) + aoff;
#pragma unroll
        for (int s = 0; s < NS; ++s) {
          store_piece(s, v[s]);
          if (b == 0 && s == 0 && si == 0) MLORA_STAMP(4);  // shrink: first piece arrived and is on its way to LDS
          if (An) request_piece(An, s, v[s]);
          __syncthreads();
          if (active) {
#pragma unroll
            for (int i = s * KSS; i < (s + 1) * KSS; ++i) {
#pragma unroll
              for (int rb = 0; rb < RB; ++rb) {
                if constexpr (MASKED) {
                  if (rb >= rb_n) continue;
                }
                const int rr = rb * 16 + lr;
                Pack8 aw;
                aw.raw = *reinterpret_cast<const i32x4*>(&s_a[(rr < R ? rr : R - 1) * ASTRIDE + i * 32 + lg * 8]);
                acc[rb] = Mma<T>::run(aw, xa[i], acc[rb]);
              }
            }
            if constexpr (MASKED) {
              if (s == NS - 1) mfma_settle(acc);  // rank blocks were skipped by branches
            }
          }
        }
        if (active && b + 1 < nbatch) {
#pragma unroll
          for (int s = 0; s < NS; ++s) request_x_piece((b + 1) * XW, s);
        }
      }
      if (si == 0) MLORA_STAMP(5);  // shrink: first slice multiplied
      write_partials(acc, si);
    }
    return;
  }

  // (Written once for wavefronts whose token block exists and once for those without one, which
  // only help with the slabs: a branch on `active` around the x requests keeps the compiler from
  // counting the loads in flight, and the wait for a slab then is a wait for the x batch requested
  // after it as well.)
  auto batches = [&](auto act_tag) {
  constexpr bool ACT = decltype(act_tag)::value;
  Pack8 xa[XK], xb[DB ? XK : 1];
  f32x4 acc[RB];
  bool first = true;
  // One x batch: `cur` holds it (or is about to), `nxt` receives the following one meanwhile.
  auto run_batch = [&](Pack8(&cur)[XK], Pack8(&nxt)[XK], int si, int b) {
    const T* A = static_cast<const T*>(sl.a[slice0 + si]) + aoff;
    if (DB && ACT && b + 1 < nbatch) request_x(nxt, (b + 1) * XW);
#pragma unroll
    for (int s = 0; s < SPB; ++s) {
      if (!first) __syncthreads();  // everyone is done reading the previous slab
      first = false;
      store_slab();
      if (b == 0 && s == 0 && si == 0) MLORA_STAMP(4);  // shrink: first slab arrived and is on its way to LDS
      __syncthreads();
      // the slab after this one: same batch, next batch, or the first of the next slice
      if (s + 1 < SPB) request_slab(A + b * XW + (s + 1) * KR);
      else if (b + 1 < nbatch) request_slab(A + (b + 1) * XW);
      else if (si + 1 < nsl) request_slab(static_cast<const T*>(sl.a[slice0 + si + 1]) + aoff);
      if (ACT) {
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
        if constexpr (MASKED) {
          if (s == SPB - 1) mfma_settle(acc);  // rank blocks were skipped by branches
        }
      }
    }
    if (!DB && ACT && b + 1 < nbatch) request_x(cur, (b + 1) * XW);
  };

  request_slab(static_cast<const T*>(sl.a[slice0]) + aoff);
  if (ACT) request_x(xa, 0);
  MLORA_STAMP(3);  // shrink: first slab and first x batch requested (the token rows are here)
  for (int si = 0; si < nsl; ++si) {
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) acc[rb] = f32x4{0.f, 0.f, 0.f, 0.f};
    if constexpr (DB) {
      // Two x buffers, one slab per batch.  A batch that has a successor (MORE) requests the
      // successor's x batch, waits for its own slab alone, and requests the successor's slab
      // after the barrier; the last batch of the K part is a copy of its own without those
      // requests.  Written that way (instead of tests on b inside one body) every wait counts
      // the requests younger than what it waits for: the x batch that was just requested stays
      // in flight while the current one is multiplied.
      auto batch = [&](auto more_tag, Pack8(&cur)[XK], Pack8(&nxt)[XK], int b) __attribute__((always_inline)) {
        constexpr bool MORE = decltype(more_tag)::value;
        static_assert(SPB == 1, "one slab per batch");
        const T* A = static_cast<const T*>(sl.a[slice0 + si]) + aoff;
        if (MORE && ACT) request_x(nxt, (b + 1) * XW);
        __syncthreads();  // everyone is done reading the previous slab
        store_slab();
        if (b == 0 && si == 0) MLORA_STAMP(4);  // shrink: first slab arrived and is on its way to LDS
        __syncthreads();
        if constexpr (MORE) request_slab(A + (b + 1) * XW);
        else if (si + 1 < nsl) request_slab(static_cast<const T*>(sl.a[slice0 + si + 1]) + aoff);
        if (ACT) {
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
              acc[rb] = Mma<T>::run(aw, cur[i], acc[rb]);
            }
          }
          if constexpr (MASKED && !MORE) mfma_settle(acc);  // rank blocks were skipped by branches
        }
      };
      int b = 0;
      for (; b + 2 < nbatch; b += 2) {
        batch(std::true_type{}, xa, xb, b);
        batch(std::true_type{}, xb, xa, b + 1);
      }
      if (b + 1 < nbatch) {
        batch(std::true_type{}, xa, xb, b);
        batch(std::false_type{}, xb, xa, b + 1);
      } else {
        batch(std::false_type{}, xa, xb, b);
      }
    } else {
      for (int b = 0; b < nbatch; ++b) run_batch(xa, xa, si, b);
    }
    if (si == 0) MLORA_STAMP(5);  // shrink: first slice multiplied
    if (ACT || TO_LDS) write_partials(acc, si);  // (to LDS: wavefronts without tokens enter zeros)
  }
  };
  if (active) batches(std::true_type{});
  else batches(std::false_type{});
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

// y is touched once per launch (a non-temporal hint on its accesses measured no gain).  An item
// stays the raw vectors it was fetched as until it is used: unpacked where it is requested, its
// arithmetic is scheduled ahead of the barrier that ends the staging of the intermediate, and the
// wavefront waits for the item in front of work that could have run meanwhile.
template <typename T, int N>
__device__ __forceinline__ typename YRaw<N>::type load_y(const T* p) {
  return *reinterpret_cast<const typename YRaw<N>::type*>(p);
}
template <typename T, int N>
__device__ __forceinline__ YVec<T, N> unpack_y(const typename YRaw<N>::type& r) {
  YVec<T, N> v;
  __builtin_memcpy(&v, &r, sizeof(r));
  return v;
}
template <typename T, int N>
__device__ __forceinline__ void store_y(T* p, const YVec<T, N>& v) {
  typedef typename YRaw<N>::type Raw;
  Raw r;
  __builtin_memcpy(&r, &v, sizeof(r));
  *reinterpret_cast<Raw*>(p) = r;
}

// Body of the expand for the tiles of one workgroup.  MASKED: some tile's slot holds an adapter of
// fewer ranks than the buffers: chunks of the intermediate the shrink did not write are not read,
// ranks at or above the adapter's are zero in the intermediate, B columns from that rank on are
// not fetched (zeros take their place in the operand).  The unmasked instance is the code without
// any of those tests.
//
// SC1: the partial sums are fetched with agent-scope loads (past the compute unit's and the XCD's
// caches): they were written by other workgroups of the same launch.
//
// PRE: the intermediate of the (one) tile is in `s_h` already, put there by this workgroup.
template <typename T, int R, int CPL, int TPF, int G, bool MASKED, bool SC1 = false, bool PRE = false>
__device__ __forceinline__ void expand_body(T* __restrict__ s_h, int* __restrict__ s_row, int* __restrict__ s_slot, int* __restrict__ s_m,
                                            int* __restrict__ s_eff, const int32_t* __restrict__ plan, const float* __restrict__ hws,
                                            void* __restrict__ yv_, int64_t ys, int T_, int num_slices, int ksplit,
                                            float scaling, const ExpandSplit& sp, const int (&slot)[G], const int (&start)[G],
                                            const int (&m)[G], const int (&eff)[G], const int (&rowv)[G]) {
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

  // The partial sums of a tile's intermediate: requested (every K part together), then summed,
  // scaled, split and written to LDS.  The first tile's are requested before anything else: they
  // depend on the tile record alone, and are on their way while the token rows make theirs.
  const int64_t hrow = static_cast<int64_t>(num_slices) * R;
  const int64_t part = static_cast<int64_t>(T_) * hrow;
  f32x4 t[HC][kMaxKSplit][2];
  auto request_h = [&](int g) {
    const float* src = hws + static_cast<int64_t>(start[g]) * hrow + sp.slice * R;
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
          if (used && SC1) {
            const uint64_t* q8 = reinterpret_cast<const uint64_t*>(q + kp * part);
#pragma unroll
            for (int w = 0; w < 4; ++w) {
              const uint64_t pair = __hip_atomic_load(q8 + w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
              t[h][kp][w >> 1][2 * (w & 1)] = __uint_as_float(static_cast<uint32_t>(pair));
              t[h][kp][w >> 1][2 * (w & 1) + 1] = __uint_as_float(static_cast<uint32_t>(pair >> 32));
            }
          } else if (used) {
            t[h][kp][0] = *reinterpret_cast<const f32x4*>(q + kp * part);
            t[h][kp][1] = *reinterpret_cast<const f32x4*>(q + kp * part + 4);
          } else {
            t[h][kp][0] = f32x4{0.f, 0.f, 0.f, 0.f};
            t[h][kp][1] = f32x4{0.f, 0.f, 0.f, 0.f};
          }
        }
      }
    }
  };
  auto stage_h = [&](int g) {
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
  };

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
  int first_step = 0;  // (set once the tiles' sizes are in LDS)
  auto column = [&](int c0) {  // first of this lane's CPL columns, clamped into the range
    const int c = c0 + CPL * lr;
    return c < sp.n1 ? c : sp.n1 - 8;
  };
  typedef typename YRaw<CPL>::type YItem[TPF][4];  // a y item as it was fetched: 16 * TPF tokens x 16 * CPL columns of a wavefront
  auto issue_y = [&](YItem& buf, int c0, int st) {
    const int g = st / NB, tp = (st % NB) * TPF, cl = column(c0);
#pragma unroll
    for (int u = 0; u < TPF; ++u) {
      const i32x4 rows = *reinterpret_cast<const i32x4*>(&s_row[g * MLORA_TILE_BIG + (tp + u) * 16 + 4 * lg]);
#pragma unroll
      for (int i = 0; i < 4; ++i) buf[u][i] = load_y<T, CPL>(ybase + static_cast<int64_t>(rows[i]) * ys + cl);
    }
  };
  Pack8 bop[CPL][KSTEPS];
  int b_slot = -1, b_c0 = -1;  // what bop holds
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
  };
  auto process = [&](YItem& buf, int c0, int st) {
    const int g = st / NB, tp = (st % NB) * TPF;
    const int mg = s_m[g];
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
          out[j] = Mma<T>::run(hlo[ks], bop[j][ks], out[j]);
          out[j] = Mma<T>::run(hop[ks], bop[j][ks], out[j]);
        }
      }
      // lane holds out[token 16*tb + 4*lg + i][column c0 + CPL*lr + j]
      const i32x4 rows = *reinterpret_cast<const i32x4*>(&s_row[g * MLORA_TILE_BIG + tb * 16 + 4 * lg]);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (col_ok && tb * 16 + 4 * lg + i < mg) {
          const YVec<T, CPL> yv = unpack_y<T, CPL>(buf[u][i]);
          YVec<T, CPL> r;
#pragma unroll
          for (int j = 0; j < CPL; ++j) r.e[j] = from_f32<T>(to_f32(yv.e[j]) + out[j][i]);
          store_y<T, CPL>(ybase + static_cast<int64_t>(rows[i]) * ys + c, r);
        }
      }
    }
  };

  YItem ya, yb;
  int c0 = sp.n0 + wave * SPAN;
  const bool has_work = c0 < sp.n1;

  // `rowv[g]` (threads 0..63): token row at position tid of tile g, requested by the caller
  // together with the tile records.  Entries past the end of a tile name valid rows too (a
  // valid row to read, never written).  The partial sums of the first tile hang on the tile
  // record alone; they are requested before the barrier the rows pass through, so that they and
  // the y rows are on their way together.  (The B rows of the first span could go out there too,
  // but they are 16 KB per wavefront and hold everything behind them up: prefill 3748 -> 3858 us.)
#pragma unroll
  for (int g = 0; g < G; ++g) {
    if (tid == 0) { s_slot[g] = slot[g]; s_m[g] = m[g]; s_eff[g] = eff[g]; }
    if (m[g] > 0 && tid < MLORA_TILE_BIG) s_row[g * MLORA_TILE_BIG + tid] = rowv[g];
  }
  if constexpr (!PRE) {
    if (m[0] > 0) request_h(0);
  }
  __syncthreads();
  if constexpr (!SC1) MLORA_STAMP(10);  // expand: token rows (and the first partial sums) here
  first_step = next_step(-1);  // exists: some tile holds tokens
  int st = first_step;
  auto advance = [&](int fc0, int fst, int& nc0, int& nst) {  // item after (fc0, fst); false when there is none
    nst = next_step(fst);
    nc0 = fc0;
    if (nst >= STEPS) {
      nst = first_step;
      nc0 = fc0 + kExpandWaves * SPAN;
    }
    return nc0 < sp.n1;
  };
  // H tiles -> LDS: K partials summed (always in the same order), scaled, split into leading
  // part and remainder; absent tokens get zeros.  All loads of a tile are in flight together.
  auto stage_all = [&]() {
    if constexpr (PRE) return;
#pragma unroll
    for (int g = 0; g < G; ++g) {
      if (m[g] == 0) continue;
      if (g > 0) request_h(g);
      stage_h(g);
    }
  };
  // the B rows of an item's span and slot, if the registers do not hold them already
  auto ensure_b = [&](int c0, int st) {
    const int g = st / NB, sg = s_slot[g];
    if (sg != b_slot || c0 != b_c0) load_b(c0, sg, s_eff[g]);
  };
  // The B rows and the first two y items go out, then the intermediate is staged while they are
  // on their way.  The staging is written out once per path (no work / one item / two items) so
  // that each is straight-line code from the requests to the staging: the compiler then waits for
  // the partial sums alone, not for everything requested after them.
  // (Every path passes the one barrier that ends the staging in its own copy: a wavefront counts
  // at the barrier wherever its program counter is.  The markers keep the compiler from merging
  // the ends of the copies into one block, where it would have to wait for every load again.)
  if (!has_work) {
    stage_all();
    asm volatile("; staged, no item" ::: "memory");
    __syncthreads();
    if constexpr (!SC1) MLORA_STAMP(11);  // expand: intermediate in LDS
    return;
  }
  int c1 = 0, st1 = 0;
  load_b(c0, s_slot[st / NB], s_eff[st / NB]);
  issue_y(ya, c0, st);
  if (!advance(c0, st, c1, st1)) {
    stage_all();
    asm volatile("; staged behind one item" ::: "memory");
    __syncthreads();
    if constexpr (!SC1) MLORA_STAMP(11);
    process(ya, c0, st);
    if constexpr (!SC1) MLORA_STAMP(14);  // expand: wavefront 0 has stored its first item
    if constexpr (!SC1) MLORA_STAMP(12);  // expand: wavefront 0 has stored an item (the last stamp taken stays)
  } else {
    issue_y(yb, c1, st1);
    stage_all();
    asm volatile("; staged behind two items" ::: "memory");
    __syncthreads();
    if constexpr (!SC1) MLORA_STAMP(11);
    // Two y buffers, used in turn, both on their way whenever the wavefront has two more items.
    // The order inside the loop is what lets the compiler count the loads in flight instead of
    // waiting for all of them: an item's B rows are looked after (a reload only when span or slot
    // change, behind a branch) BEFORE the item after it is requested, so whatever waits for B
    // rows or for a y item knows how many requests are younger; the paths that run out of items
    // leave the loop where they find out, with their own copy of the last step.
    process(ya, c0, st);
    if constexpr (!SC1) MLORA_STAMP(14);
    if constexpr (!SC1) MLORA_STAMP(12);
    for (;;) {
      // here: (c1, st1) is on its way in yb; ya is free
      int c2, st2;
      const bool more2 = advance(c1, st1, c2, st2);
      ensure_b(c1, st1);
      if (!more2) {
        process(yb, c1, st1);
        if constexpr (!SC1) MLORA_STAMP(12);
        break;
      }
      issue_y(ya, c2, st2);
      process(yb, c1, st1);
      if constexpr (!SC1) MLORA_STAMP(12);
      // here: (c2, st2) is on its way in ya; yb is free
      const bool more3 = advance(c2, st2, c1, st1);
      ensure_b(c2, st2);
      if (!more3) {
        process(ya, c2, st2);
        if constexpr (!SC1) MLORA_STAMP(12);
        break;
      }
      issue_y(yb, c1, st1);
      process(ya, c2, st2);
      if constexpr (!SC1) MLORA_STAMP(12);
    }
  }
#ifdef MLORA_TRACE
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  if constexpr (!SC1) MLORA_STAMP(13);  // expand: wavefront 0's stores acknowledged
#endif
}

// The fp32 partials of the intermediate live behind the head of the workspace.
float* partials_of(const MloraAddArgs* a) { return reinterpret_cast<float*>(static_cast<char*>(a->workspace) + MLORA_WORKSPACE_HEAD_BYTES); }
size_t partials_room(const MloraAddArgs* a) {
  return a->workspace_bytes > MLORA_WORKSPACE_HEAD_BYTES ? static_cast<size_t>(a->workspace_bytes) - MLORA_WORKSPACE_HEAD_BYTES : 0;
}

// Diagnostic knobs, read from the environment once and again after mlora_reload_knobs().
struct SgmvKnobs {
  int generation = -1, kr, ksplit, all_slices, xdb, group, wgs, nt, cpl;
  void read() {
    generation = knob_generation();
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

// One fp32 partial of the intermediate: [T, slices, r].
inline size_t partial_bytes(int num_tokens, int num_slices, int r) {
  return static_cast<size_t>(num_tokens) * static_cast<size_t>(num_slices) * static_cast<size_t>(r) * sizeof(float);
}

// How a call is cut into work, shared by the two-launch and the one-launch form.
struct SgmvShape {
  bool empty;
  PlanLayout lay;
  ShrinkSlices sl;
  int tiles8;     // tiles / 8: 64-token tiles of the long segments, then the short segments
  int big_cap;    // tiles below this index are 64-token tiles
  int kr, xw;     // shrink: A slab width, x batch width
  int ksplit, krange, all_slices;
  int group;      // expand: consecutive 64-token tiles per workgroup
  int cpl;        // expand: columns per lane
  int nsplit;     // expand: column ranges
  int big_units;  // expand: groups of 64-token tiles
  int units;      // expand: those plus the short segments
  ExpandSplits splits;
};

// one_launch: the cut for the form whose workgroups do both products (256-column slabs and batches,
// which leave the registers the kernel needs besides; as many shrink roles per unit as it has workgroups).
inline SgmvShape sgmv_shape(const MloraAddArgs* a, bool one_launch = false) {
  SgmvShape s;
  s.empty = true;
  s.lay = plan_layout(a->num_tokens, a->num_slots);
  s.big_cap = (s.lay.cap_big + 7) & ~7;
  int short_cap = a->num_slots < a->num_tokens ? a->num_slots : a->num_tokens;  // a short segment is one small tile
  if (short_cap > s.lay.cap_small) short_cap = s.lay.cap_small;
  const int cap = s.big_cap + ((short_cap + 7) & ~7);
  if (cap == 0) return s;
  s.tiles8 = cap / 8;
  int cols = 0;
  for (int i = 0; i < a->num_slices; ++i) {
    cols += a->slices[i].n;
    s.sl.a[i] = a->slices[i].a;
  }
  for (int i = a->num_slices; i < MLORA_MAX_SLICES; ++i) s.sl.a[i] = nullptr;
  if (cols == 0) return s;
  s.empty = false;
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
    // (a workgroup per compute unit, and K parts of at most 1024 columns: on the prefill batch
    // gate_up with one part takes 72.2 us per call against 73.3 with two, o with two 19.6
    // against 22.4 with one, down with four 33.6 against 35.7 with two and 50.5 with one)
    while (ksplit < kMaxKSplit && a->k % (xw * ksplit * 2) == 0 &&
           (static_cast<long long>(est_tiles) * a->num_slices * ksplit < 256 || a->k / ksplit > 1024))
      ksplit *= 2;
  }
  if (ksplit > max_parts) ksplit = max_parts;
  if (ksplit > kMaxKSplit) ksplit = kMaxKSplit;
  while (ksplit > 1 && a->k % (xw * ksplit) != 0) --ksplit;
  // three or more slices: one workgroup walks them all with the x rows it already holds, when
  // its K part is a single batch (measured on the prefill batch: qkv 31.9 -> 29.6 us per call;
  // with two slices the shorter chain of separate workgroups wins, gate_up 76.6 vs 77.8)
  s.all_slices = 0;
  if (a->num_slices >= sgmv_knobs().all_slices) {
    const int parts = a->k / xw;
    if (parts <= kMaxKSplit && parts <= max_parts) {
      ksplit = parts;
      s.all_slices = 1;
    }
  }
  s.ksplit = ksplit;
  s.krange = a->k / ksplit;
  // a K part of several batches: the form with two x buffers (256-column batches)
  if (xw == 512 && s.krange > xw && sgmv_knobs().xdb) { xw = 256; kr = 256; }
  s.kr = kr;
  s.xw = xw;

  // expand: consecutive tiles per workgroup (they share their B rows when they share their
  // slot), then column ranges so that the grid has about 2048 workgroups
  int group = sgmv_knobs().group;
  // wide projections only: narrow ones need the workgroups.  Two tiles per workgroup, not four: on
  // the prefill batch (8 adapters) gate_up takes 72.2 against 73.2 us per call, on the mixed batch
  // (126 adapters, many of them with fewer than four tiles) 105.8 against 110.4
  if (group != 1 && group != 2 && group != 4) group = (cols >= 4096 && est_tiles >= 64) ? 2 : 1;
  if (one_launch && group == 2) group = 4;  // the one-launch kernel exists for one tile and for four
  const int target = sgmv_knobs().wgs;
  int nt = sgmv_knobs().nt;
  if (nt <= 0) {
    const long long want = static_cast<long long>(cols) * (est_tiles / group + 1) / (target > 0 ? target : 1);
    nt = want > 8192 ? 8192 : static_cast<int>(want);
  }
  s.group = group;
  s.nsplit = fill_splits(a, nt, s.splits.split);
  s.cpl = sgmv_knobs().cpl == 4 ? 4 : 8;
  if (one_launch && a->k % 256 == 0) {
    // the unit's workgroups (one per column range) share out its shrink roles (tile, slice, K part):
    // about one role each
    s.kr = s.xw = 256;
    s.all_slices = 0;
    if (group * a->num_slices > s.nsplit) s.group = group = 1;  // every slice has a column range: one role each at least
    int parts = sgmv_knobs().ksplit;
    if (parts <= 0) {
      parts = 1;
      while (parts < kMaxKSplit && group * a->num_slices * parts * 2 <= s.nsplit && a->k % (256 * parts * 2) == 0) parts *= 2;
    }
    if (parts > max_parts) parts = max_parts;
    if (parts > kMaxKSplit) parts = kMaxKSplit;
    while (parts > 1 && (a->k % (256 * parts) != 0 || group * a->num_slices * parts > s.nsplit)) --parts;
    s.ksplit = parts;
    s.krange = a->k / parts;
  }
  s.big_units = s.big_cap / group;  // big_cap is a multiple of 32: a multiple of 8 again
  s.units = s.big_units + (s.tiles8 * 8 - s.big_cap);
  return s;
}

}  // namespace

}  // namespace mlora
