// Computes, for prefill-sized batches and in ONE launch, what the reference computes with its
// segment-grouped shrink kernel, a temporary [slices, T, r] tensor and its expand kernel
// (nanovllm_voxcpm/lora.py:291-381 driving lora_ops/triton_ops/lora_shrink_op.py:16-101, 257-341 and
// lora_expand_op.py:11-170): y_i[t] += (x[t] . A_i[s_t]^T) . B_i[s_t]^T * scaling, tokens grouped by slot.
//
// The work is cut as in the two-launch form (sgmv.hip): a unit is a group of G consecutive
// 64-token tiles of the long segments, or one short segment; the shrink of a unit consists of
// roles (tile of the group, slice, K part) and its expand of column ranges.  Here one grid
// (8, column ranges, units / 8) does both: the workgroups of a unit first share out the unit's
// shrink roles among themselves, write the fp32 partial sums to the workspace and, once those
// stores have been acknowledged by the L2, seal each finished role with the unit's tag and the
// XCD they ran on; then each waits for the seals of the roles its own slice needs and expands
// its column range, fetching the partial sums past its compute unit's L1 (agent-scope loads)
// from that same L2.  No kernel boundary and no
// drained machine between the two products, and the expand's workgroups are already resident
// when the intermediate arrives.
//
// Waiting is safe and bounded.  Workgroups are dispatched in the order of their linear index and
// the members of a unit are consecutive there (blockIdx.x, the XCD, is fixed for a unit), so
// whenever a member waits, every unit before its own is completely resident or finished and
// will free its compute-unit slots without outside help; a unit's members wait only for each
// other.  Should a seal still be missing after `spin_ticks` (or the workspace head be
// uninitialised), the waiting workgroup computes the missing roles itself: the same arithmetic in
// the same order, so the words it writes are the ones the late producer writes.  The last
// workgroup of the grid to finish advances the workspace's generation, which makes every seal of
// this launch stale.
#include "sgmv_body.h"

namespace mlora {

namespace {

constexpr int kFusedThreads = 256;
static_assert(kFusedThreads == kShrinkWaves * kWave && kFusedThreads == kExpandWaves * kWave, "both products run with four wavefronts");


// The two products as functions of their own (not inlined into the kernel): each gets the register
// file to itself, as in the two-launch form, instead of one allocation that has to carry the
// kernel's state through both.
template <typename T, int R, int KR, int XW, bool DB>
__device__ __forceinline__ void fused_shrink_role(T* __restrict__ s_a, const int32_t* __restrict__ plan, const void* __restrict__ xv, float* __restrict__ hws, int64_t xs, int sorted_off,
                                                            int T_, int K, int num_slices, int krange, int all_slices, const ShrinkSlices& sl,
                                                            int slice0, int kpart, int slot, int start, int m, int eff) {
  // token row of this lane (positions past the end of the tile repeat its last token)
  const int ti = (threadIdx.x / kWave) * 16 + (threadIdx.x & 15);
  const int row = plan[sorted_off + start + (ti < m ? ti : m - 1)];
  if (R > 16 && ((eff + 15) >> 4) < (R + 15) / 16)
    shrink_body<T, R, KR, XW, DB, true, false>(s_a, xv, hws, xs, T_, K, num_slices, krange, all_slices, sl, slice0, kpart, slot, start, m, eff, row);
  else
    shrink_body<T, R, KR, XW, DB, false, false>(s_a, xv, hws, xs, T_, K, num_slices, krange, all_slices, sl, slice0, kpart, slot, start, m, eff, row);
}

// The same for the roles a workgroup computes because their seals did not arrive: the exception, so
// a function of its own (called in a loop) rather than a second inlined copy.
template <typename T, int R, int KR, int XW, bool DB>
__device__ __attribute__((noinline)) void fused_shrink_role_late(T* s_a, const int32_t* plan, const void* xv, float* hws, int64_t xs, int sorted_off,
                                                                 int T_, int K, int num_slices, int krange, int all_slices, const ShrinkSlices& sl,
                                                                 int slice0, int kpart, int slot, int start, int m, int eff) {
  fused_shrink_role<T, R, KR, XW, DB>(s_a, plan, xv, hws, xs, sorted_off, T_, K, num_slices, krange, all_slices, sl, slice0, kpart, slot, start, m, eff);
}

template <typename T, int R, int CPL, int TPF, int G>
__device__ __forceinline__ void fused_expand(T* s_h, int* s_row, int* s_slot, int* s_m, int* s_eff, const int* s_start,
                                                       const int32_t* plan, const float* hws, void* yv_, int64_t ys, int sorted_off, int T_,
                                                       int num_slices, int ksplit, float scaling, const ExpandSplit& sp) {
  int slot[G], start[G], m[G], eff[G], rowv[G];
  bool masked = false;
#pragma unroll
  for (int g = 0; g < G; ++g) {
    slot[g] = s_slot[g]; start[g] = s_start[g]; m[g] = s_m[g]; eff[g] = s_eff[g];
    masked |= m[g] > 0 && eff[g] < R;
    // token row at position tid of the tile (positions past its end repeat its last token)
    const int tid = threadIdx.x;
    rowv[g] = (m[g] > 0 && tid < MLORA_TILE_BIG) ? plan[sorted_off + start[g] + (tid < m[g] ? tid : m[g] - 1)] : 0;
  }
  __syncthreads();  // expand_body rewrites the arrays read above
  if (masked)
    expand_body<T, R, CPL, TPF, G, true, true>(s_h, s_row, s_slot, s_m, s_eff, plan, hws, yv_, ys, T_, num_slices, ksplit, scaling, sp, slot, start,
                                               m, eff, rowv);
  else
    expand_body<T, R, CPL, TPF, G, false, true>(s_h, s_row, s_slot, s_m, s_eff, plan, hws, yv_, ys, T_, num_slices, ksplit, scaling, sp, slot, start,
                                                m, eff, rowv);
}

template <typename T, int R, int KR, int XW, bool DB, int CPL, int TPF, int G>
__global__ __launch_bounds__(kFusedThreads, 2) void sgmv_fused_kernel(
    const int32_t* __restrict__ plan, const void* __restrict__ xv, void* __restrict__ yv_, uint32_t* __restrict__ ws,
    float* __restrict__ hws, int64_t xs, int64_t ys, int big_off, int small_off, int big_units, int sorted_off, int T_, int K,
    int num_slots, int num_slices, int ksplit, int krange, int all_slices, float scaling, int spin_ticks, int trusted,
    const int32_t* __restrict__ eff_rank, ShrinkSlices sl, ExpandSplits splits) {
  constexpr int HSTRIDE = 2 * R + 8;
  constexpr int kShrinkLds = R * (KR + 8) * static_cast<int>(sizeof(T));
  constexpr int kExpandLds = G * MLORA_TILE_BIG * HSTRIDE * static_cast<int>(sizeof(T));
  constexpr int kLds = kShrinkLds > kExpandLds ? kShrinkLds : kExpandLds;
  // the A slabs of the shrink and the staged intermediate of the expand use the same LDS in turn
  __shared__ __attribute__((aligned(16))) unsigned char s_raw[kLds];
  __shared__ __attribute__((aligned(16))) int s_row[G * MLORA_TILE_BIG];
  __shared__ int s_slot[G], s_m[G], s_eff[G], s_start[G];
  __shared__ uint32_t s_todo[2];
  T* const s_a = reinterpret_cast<T*>(s_raw);
  T* const s_h = reinterpret_cast<T*>(s_raw);

  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int unit = tile_position(big_units);  // blockIdx.x is the XCD; a block of the list of units is G positions of the XCD's block of tiles
  const int c = blockIdx.y, W = gridDim.y;
  const bool is_big = unit < big_units;
  const int sidx = is_big ? 0 : unit - big_units;
  MLORA_STAMP(0);  // first instruction

  // ---- round trip 1: header, every candidate record, the unit's generation -----------------------
  const i32x4 hdr0 = *reinterpret_cast<const i32x4*>(plan);
  const i32x4 hdr1 = *reinterpret_cast<const i32x4*>(plan + 4);
  const i32x4 hdr2 = *reinterpret_cast<const i32x4*>(plan + 8);
  const i32x4 small = *reinterpret_cast<const i32x4*>(plan + small_off + sidx * MLORA_SMALL_TILE_WORDS);
  i32x4 big[G];
#pragma unroll
  for (int g = 0; g < G; ++g) big[g] = reinterpret_cast<const i32x4*>(plan + big_off)[is_big ? unit * G + g : 0];
  const ExpandSplit sp = splits.split[c];
  const uint32_t signature = ws[0];
  // {generation, arrivals} of the workspace: one pair for the whole launch, so that every seal any
  // earlier launch left anywhere (whatever its layout was) carries a tag below this launch's
  uint32_t* const ustate = ws + kWsTileOff / 4;
  const uint32_t tag = ustate[0] + 1u;
  const uint32_t arrivals0 = ustate[1], gen_check = ustate[2];
  const int n_short = hdr1[MLORA_PLAN_TILES_SHORT - 4];
  int slot[G], start[G], m[G], any = 0;
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const bool have = is_big ? true : (g == 0 && sidx < n_short);  // (places of the list of 64-token tiles that hold none carry count 0)
    slot[g] = is_big ? big[g][0] : small[0];
    start[g] = is_big ? big[g][1] : small[2];
    m[g] = is_big ? big[g][2] : small[1];
    if (!have || m[g] <= 0 || slot[g] < 0 || slot[g] >= num_slots) m[g] = 0;
  }
  // rank of the adapter in each tile's slot (a second, dependent fetch, only with the vector given)
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
  // One exit test, the same for every workgroup of a unit
  const int usable = int(hdr0[MLORA_PLAN_MAGIC] == MLORA_PLAN_MAGIC_VALUE) & int(hdr0[MLORA_PLAN_NUM_TOKENS] == T_) &
                     int(hdr0[MLORA_PLAN_MAX_SLOTS] == num_slots) & int(any > 0);
  // seals and generations can be used: the head is in the state a launch (or the initialisation) left it in
  const bool xok = trusted | ws_state_ok(signature, tag - 1u, arrivals0, gen_check, gridDim.x * gridDim.y * gridDim.z);
  // every workgroup of the grid reports exactly once that it is done (also the ones without work);
  // the last one advances the generation, which makes every seal of this launch stale
  auto count_done = [&]() {
    if (xok && tid == 0) {
      const uint32_t before = __hip_atomic_fetch_add(ustate + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (before + 1u == gridDim.x * gridDim.y * gridDim.z) {
        const uint32_t next = tag == 0xffffffffu ? 0u : tag;  // generation + 1, the next tag, is never 0
        __hip_atomic_store(ustate + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(ustate + 2, next ^ kWsGenCheck, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(ustate, next, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  };
  if (!usable) {
    count_rejected_plan(plan, hdr0[MLORA_PLAN_MAGIC] == MLORA_PLAN_MAGIC_VALUE && hdr0[MLORA_PLAN_NUM_TOKENS] == T_ &&
                                  hdr0[MLORA_PLAN_MAX_SLOTS] == num_slots);
    count_done();
    return;
  }
  MLORA_STAMP(1);  // records, ranks and generation are here

  if (tid == 0) {
#pragma unroll
    for (int g = 0; g < G; ++g) { s_slot[g] = slot[g]; s_m[g] = m[g]; s_eff[g] = eff[g]; s_start[g] = start[g]; }
  }
  __syncthreads();

  // ---- the unit's shrink roles ------------------------------------------------------------------------
  // role s = (tile g of the group, q): q is a K part when a workgroup walks all slices, else (slice, K part)
  const int rpt = all_slices ? ksplit : num_slices * ksplit;
  const int YS = G * rpt;  // <= 64 (host)
  // a seal: {tag, XCD the sealing workgroup ran on}.  The partial sums are ordinary stores, which
  // come to rest in the L2 of the writer's XCD; only a reader on the same XCD finds them there, so
  // a seal from another XCD never matches (its reader then computes the role itself).
  uint64_t* const seals = reinterpret_cast<uint64_t*>(ws + kWsSealOff / 4) + unit * YS;  // (unit + 1) * YS seals fit the area (host)
  const uint64_t seal = (static_cast<uint64_t>(xcc_id()) << 32) | tag;
  // Role s of the unit is computed by its workgroup s (there are at least as many workgroups as
  // roles: host); `need`: the roles this workgroup's slice is made of.
  const int my_g = c / rpt;
  const bool have_role = c < YS && __builtin_amdgcn_readfirstlane(s_m[c < YS ? my_g : 0]) > 0;
  uint64_t need = 0;
  for (int s = 0; s < YS; ++s) {
    const int g = s / rpt, q = s - g * rpt;
    if (__builtin_amdgcn_readfirstlane(s_m[g]) <= 0) continue;
    if (all_slices || q / ksplit == sp.slice) need |= 1ull << s;
  }
  const uint64_t mine = have_role ? 1ull << c : 0;

  if (have_role) {
    const int q = c - my_g * rpt;
    const int slice0 = all_slices ? 0 : q / ksplit, kpart = all_slices ? q : q % ksplit;
    // (the same for every lane: kept in scalar registers, and with them every address derived from them)
    const int gs = __builtin_amdgcn_readfirstlane(s_slot[my_g]), gm = __builtin_amdgcn_readfirstlane(s_m[my_g]);
    const int ge = __builtin_amdgcn_readfirstlane(s_eff[my_g]), gstart = __builtin_amdgcn_readfirstlane(s_start[my_g]);
    fused_shrink_role<T, R, KR, XW, DB>(s_a, plan, xv, hws, xs, sorted_off, T_, K, num_slices, krange, all_slices, sl, slice0, kpart, gs, gstart,
                                        gm, ge);
  }
  MLORA_STAMP(10);  // own role multiplied, its stores issued
  // the partial sums written above have been acknowledged by the L2 ...
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  MLORA_STAMP(11);  // ... by every wavefront
  // ... and only then is the role sealed
  if (xok && have_role && tid == 0) __hip_atomic_store(seals + c, seal, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

  // ---- wait for the roles this workgroup's slice needs --------------------------------------------------
  if (wave == 0) {
    uint64_t missing = need & ~mine;
    if (xok && missing) {
      const bool wanted = lane < YS && ((missing >> lane) & 1);
      const long long t0 = wall_clock64();
      for (;;) {
        const uint64_t v = wanted ? __hip_atomic_load(seals + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : seal;
        missing = __builtin_amdgcn_ballot_w64(v != seal);
        if (spin_ticks < 0) missing = need & ~mine;  // test hook: never accept a seal
        if (!missing || spin_ticks < 0 || wall_clock64() - t0 >= spin_ticks) break;
        __builtin_amdgcn_s_sleep(2);
      }
      if (missing && spin_ticks > 0 && lane == 0) atomicAdd(ws + kWsTimeoutsWord, 1u);  // diagnostic: a wait ran out
    }
    if (lane == 0) {
      s_todo[0] = static_cast<uint32_t>(missing);
      s_todo[1] = static_cast<uint32_t>(missing >> 32);
    }
  }
  __syncthreads();
  MLORA_STAMP(12);  // the wait is over
  const uint64_t todo = (static_cast<uint64_t>(__builtin_amdgcn_readfirstlane(s_todo[1])) << 32) | static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(s_todo[0]));
  if (todo) {
    // seals that did not arrive (or a workspace whose head cannot be used): those roles are computed here
    for (int s = 0; s < YS; ++s) {
      if (!((todo >> s) & 1)) continue;
      const int g = s / rpt, q = s - g * rpt;
      const int slice0 = all_slices ? 0 : q / ksplit, kpart = all_slices ? q : q % ksplit;
      __syncthreads();  // every wavefront is done with the previous role's last slab
      fused_shrink_role_late<T, R, KR, XW, DB>(s_a, plan, xv, hws, xs, sorted_off, T_, K, num_slices, krange, all_slices, sl, slice0, kpart,
                                               s_slot[g], s_start[g], s_m[g], s_eff[g]);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  }
  // (every path to here ends in a barrier: the slab buffer is free for the intermediate)

  // ---- expand ---------------------------------------------------------------------------------------
  fused_expand<T, R, CPL, TPF, G>(s_h, s_row, s_slot, s_m, s_eff, s_start, plan, hws, yv_, ys, sorted_off, T_, num_slices, ksplit, scaling, sp);

  MLORA_STAMP(13);  // expanded (wavefront 0)
  count_done();
}

// Diagnostic knobs, read from the environment once and again after mlora_reload_knobs().
struct FusedKnobs {
  int generation = -1, spin_ticks;
  void read() {
    generation = knob_generation();
    spin_ticks = env_int("MLORA_FUSED_SPIN_TICKS", 50000);  // of the 100 MHz clock: 500 us
  }
};
const FusedKnobs& fused_knobs() {
  static FusedKnobs k;
  if (k.generation != knob_generation()) k.read();
  return k;
}

struct FusedLaunch {
  const MloraAddArgs* a;
  const SgmvShape* sh;
  int trusted;
};

template <typename T, int R, int KR, int XW, bool DB, int G>
void launch_fused_one(const FusedLaunch& l) {
  const MloraAddArgs* a = l.a;
  const SgmvShape& sh = *l.sh;
  dim3 grid(8, static_cast<unsigned>(sh.nsplit), static_cast<unsigned>(sh.units / 8));
  hipLaunchKernelGGL((sgmv_fused_kernel<T, R, KR, XW, DB, 8, 2, G>), grid, dim3(kFusedThreads), 0, static_cast<hipStream_t>(a->stream), a->plan,
                     a->x, a->y, static_cast<uint32_t*>(a->workspace), partials_of(a), a->x_stride, a->y_stride, sh.lay.big_off,
                     sh.lay.small_off, sh.big_units, sh.lay.sorted_off, a->num_tokens, a->k, a->num_slots, a->num_slices, sh.ksplit,
                     sh.krange, sh.all_slices, a->scaling, fused_knobs().spin_ticks, l.trusted, a->effective_rank,
                     sh.sl, sh.splits);
}

template <typename T, int R, int G>
void launch_fused_slab(const FusedLaunch& l) {
  launch_fused_one<T, R, 256, 256, true, G>(l);
}

template <typename T, int R>
void launch_fused_group(const FusedLaunch& l) {
  if (l.sh->group == 4) launch_fused_slab<T, R, 4>(l);
  else launch_fused_slab<T, R, 1>(l);
}

template <typename T>
void launch_fused_rank(const FusedLaunch& l) {
  switch (l.a->r) {
    case 8: launch_fused_group<T, 8>(l); break;
    case 16: launch_fused_group<T, 16>(l); break;
    case 32: launch_fused_group<T, 32>(l); break;
    default: launch_fused_group<T, 64>(l); break;
  }
}

// The instances that exist: 256-column slabs and batches with two x buffers; 128-bit y accesses;
// one tile or four per unit.  And what the head of the workspace has room for.
bool shape_fits(const MloraAddArgs* a, const SgmvShape& sh) {
  if (sh.empty) return true;
  const bool slab = sh.kr == 256 && sh.xw == 256 && !sh.all_slices;
  if (!slab || sh.cpl != 8 || (sh.group != 1 && sh.group != 4)) return false;
  const int roles = sh.group * (sh.all_slices ? sh.ksplit : a->num_slices * sh.ksplit);
  if (roles > 64 || roles > sh.nsplit || sh.units > kWsTiles) return false;  // one shrink role per workgroup of a unit
  return static_cast<int64_t>(sh.units) * roles * 8 <= kWsSealBytes;
}

}  // namespace

void fused_trace_set(void* buf) {
#ifdef MLORA_TRACE
  (void)hipMemcpyToSymbol(HIP_SYMBOL(trace_buf), &buf, sizeof(buf));
#else
  (void)buf;
#endif
}

bool fused_supported(const MloraAddArgs* a) {
  if (!sgmv_supported(a) || !sgmv_workspace_ok(a) || a->k % 256 != 0) return false;
  if (a->workspace_bytes < MLORA_WORKSPACE_HEAD_BYTES) return false;
  return shape_fits(a, sgmv_shape(a, true));
}

int launch_fused(const MloraAddArgs* a, bool trusted_workspace) {
  const SgmvShape sh = sgmv_shape(a, true);
  if (sh.empty) return 0;
  FusedLaunch l{a, &sh, trusted_workspace ? 1 : 0};
  if (a->dtype == MLORA_DTYPE_BF16) launch_fused_rank<__bf16>(l);
  else launch_fused_rank<_Float16>(l);
  return check_launch("mlora_add_lora(fused sgmv)");
}

}  // namespace mlora
