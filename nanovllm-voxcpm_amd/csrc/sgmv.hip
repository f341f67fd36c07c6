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
#include "sgmv_body.h"

namespace mlora {

namespace {

template <typename T, int R, int KR, int XW, bool DB>
__global__ __launch_bounds__(kShrinkWaves* kWave, 2) void sgmv_shrink_kernel(const int32_t* __restrict__ plan, const void* __restrict__ xv,
                                                                             float* __restrict__ hws, int64_t xs, int big_off,
                                                                             int small_off, int big_cap, int bigrows_off, int T_, int K,
                                                                             int num_slots, int num_slices, int ksplit, int krange,
                                                                             int all_slices, const int32_t* __restrict__ eff_rank, ShrinkSlices sl) {
  constexpr int ASTRIDE = KR + 8;  // padded LDS row: 16 rows x 16 bytes cover all banks once
  __shared__ __attribute__((aligned(16))) T s_a[R * ASTRIDE];
  // all_slices: the workgroup walks every slice of the projection with the x rows it holds in
  // registers (its K part is a single batch then), instead of one workgroup per slice
  const int slice0 = all_slices ? 0 : blockIdx.y / ksplit, kpart = all_slices ? blockIdx.y : blockIdx.y % ksplit;
  const int tile = tile_position(big_cap);  // blockIdx.x is the XCD
  MLORA_STAMP(0);  // first instruction
  const int row = tile_row(plan, bigrows_off, small_off, big_cap, tile, (threadIdx.x / kWave) * 16 + (threadIdx.x & 15));
  const TileRef tr = fetch_tile(plan, big_off, small_off, big_cap, tile, T_, num_slots);
  if (!tr.ok) {
    count_rejected_plan(plan, tr.plan_ok);
    return;
  }
  MLORA_STAMP(1);  // tile record here
  // rank of the adapter in this slot (a second, dependent fetch, only with the vector given)
  int eff = R;
  if (R > 16 && eff_rank) {
    eff = eff_rank[tr.slot];
    eff = eff < 0 ? 0 : eff > R ? R : eff;
    if (eff == 0) return;
  }
  if (R > 16 && ((eff + 15) >> 4) < (R + 15) / 16)
    shrink_body<T, R, KR, XW, DB, true>(s_a, xv, hws, xs, T_, K, num_slices, krange, all_slices, sl, slice0, kpart, tr.slot, tr.start, tr.m,
                                        eff, row);
  else
    shrink_body<T, R, KR, XW, DB, false>(s_a, xv, hws, xs, T_, K, num_slices, krange, all_slices, sl, slice0, kpart, tr.slot, tr.start, tr.m,
                                         eff, row);
#ifdef MLORA_TRACE
  MLORA_STAMP(6);  // partial sums issued
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  MLORA_STAMP(7);  // ... and acknowledged
#endif
}

template <typename T, int R, int CPL, int TPF, int G>
__global__ __launch_bounds__(kExpandWaves* kWave, 2) void sgmv_expand_kernel(const int32_t* __restrict__ plan, const float* __restrict__ hws,
                                                                             void* __restrict__ yv_, int64_t ys, int big_off, int small_off,
                                                                             int big_units, int bigrows_off, int T_, int num_slots,
                                                                             int num_slices, int ksplit, float scaling,
                                                                             const int32_t* __restrict__ eff_rank, ExpandSplits splits) {
  constexpr int HSTRIDE = 2 * R + 8;     // padded LDS row: R leading parts, R remainders
  __shared__ __attribute__((aligned(16))) T s_h[G * MLORA_TILE_BIG * HSTRIDE];
  __shared__ __attribute__((aligned(16))) int s_row[G * MLORA_TILE_BIG];
  __shared__ int s_slot[G], s_m[G], s_eff[G];

  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int lr = lane & 15, lg = lane >> 4;
  // A workgroup takes G consecutive 64-token tiles (consecutive tiles mostly belong to one slot,
  // whose B rows then stay in registers across them), or, past `big_units`, one short segment.
  const int unit = tile_position(big_units);  // blockIdx.x is the XCD; a block of the list of units is G positions of the XCD's block of tiles
  MLORA_STAMP(8);  // expand: first instruction
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
  // the token rows of the tiles: where they lie follows from the unit's number, so they are
  // requested here, with the records (threads 0..63 hold one position of every tile each)
  int rowv[G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    rowv[g] = 0;
    if (tid < MLORA_TILE_BIG) {
      if (is_big) rowv[g] = plan[bigrows_off + (unit * G + g) * MLORA_TILE_BIG + tid];
      else if (g == 0) rowv[g] = plan[small_off + sidx * MLORA_SMALL_TILE_WORDS + MLORA_SMALL_TILE_ROWS + (tid & (MLORA_TILE_SMALL - 1))];
    }
  }
  const ExpandSplit sp = splits.split[blockIdx.y];
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
  if (!usable) {
    count_rejected_plan(plan, hdr0[MLORA_PLAN_MAGIC] == MLORA_PLAN_MAGIC_VALUE && hdr0[MLORA_PLAN_NUM_TOKENS] == T_ &&
                                  hdr0[MLORA_PLAN_MAX_SLOTS] == num_slots);
    return;
  }
  MLORA_STAMP(9);  // expand: tile records here

  bool masked = false;
#pragma unroll
  for (int g = 0; g < G; ++g) masked |= m[g] > 0 && eff[g] < R;
  if (masked)
    expand_body<T, R, CPL, TPF, G, true>(s_h, s_row, s_slot, s_m, s_eff, plan, hws, yv_, ys, T_, num_slices, ksplit, scaling, sp, slot, start,
                                         m, eff, rowv);
  else
    expand_body<T, R, CPL, TPF, G, false>(s_h, s_row, s_slot, s_m, s_eff, plan, hws, yv_, ys, T_, num_slices, ksplit, scaling, sp, slot, start,
                                          m, eff, rowv);
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
                     l.lay.bigrows_off, a->num_tokens, a->k, a->num_slots, a->num_slices, l.ksplit, l.krange, l.all_slices, a->effective_rank, l.sl);
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
#define MLORA_EXPAND(CPL_, TPF_, G_)                                                                                       \
  hipLaunchKernelGGL((sgmv_expand_kernel<T, R, CPL_, TPF_, G_>), grid, dim3(kExpandWaves* kWave), 0, st, a->plan, h, a->y, \
                     a->y_stride, lay.big_off, lay.small_off, big_units, lay.bigrows_off, a->num_tokens, a->num_slots,      \
                     a->num_slices, ksplit, a->scaling, a->effective_rank, sp)
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

}  // namespace

size_t sgmv_workspace_bytes(int num_tokens, int num_slices, int r, int dtype) {
  (void)dtype;
  if (num_tokens <= 0 || num_slices <= 0 || r <= 0) return 0;
  return MLORA_WORKSPACE_HEAD_BYTES + kMaxKSplit * partial_bytes(num_tokens, num_slices, r);
}

void sgmv_trace_set(void* buf) {
#ifdef MLORA_TRACE
  (void)hipMemcpyToSymbol(HIP_SYMBOL(trace_buf), &buf, sizeof(buf));
#else
  (void)buf;
#endif
}

bool sgmv_supported(const MloraAddArgs* a) { return a->k % 128 == 0 && a->k >= 128 && exact_rank(a->r); }

// A workspace that holds at least one partial can be used (fewer K parts are taken then).
bool sgmv_workspace_ok(const MloraAddArgs* a) {
  if (!a->workspace || (reinterpret_cast<uintptr_t>(a->workspace) & 255)) return false;
  for (int i = 0; i < a->num_slices; ++i)
    if (a->slices[i].n <= 0) return false;  // every slice owns a workspace column block
  return partials_room(a) >= partial_bytes(a->num_tokens, a->num_slices, a->r);
}

// Every segment of the batch: 64-token tiles of the long ones, one short tile each for the rest.
int launch_sgmv(const MloraAddArgs* a) {
  const SgmvShape sh = sgmv_shape(a);
  if (sh.empty) return 0;
  ShrinkLaunch l;
  l.a = a; l.lay = sh.lay; l.sl = sh.sl; l.tiles8 = sh.tiles8; l.big_cap = sh.big_cap;
  l.ksplit = sh.ksplit; l.krange = sh.krange; l.all_slices = sh.all_slices;
  if (a->dtype == MLORA_DTYPE_BF16) launch_shrink_rank<__bf16>(l, sh.kr, sh.xw);
  else launch_shrink_rank<_Float16>(l, sh.kr, sh.xw);
  int rc = check_launch("mlora_add_lora(sgmv shrink)");
  if (rc) return rc;

  dim3 grid(8, static_cast<unsigned>(sh.nsplit), static_cast<unsigned>(sh.units / 8));
  if (a->dtype == MLORA_DTYPE_BF16) launch_expand_rank<__bf16>(a, sh.lay, sh.big_units, grid, sh.ksplit, sh.cpl, sh.group, sh.splits);
  else launch_expand_rank<_Float16>(a, sh.lay, sh.big_units, grid, sh.ksplit, sh.cpl, sh.group, sh.splits);
  return check_launch("mlora_add_lora(sgmv expand)");
}

}  // namespace mlora
