// Computes, for prefill-sized batches, what the reference computes with its segment-grouped
// shrink and expand kernels (nanovllm_voxcpm/lora_ops/triton_ops/lora_shrink_op.py:16-101, 257-341,
// lora_expand_op.py:11-170, kernel_utils.py:7-228, launched from nanovllm_voxcpm/lora.py:291-381):
// y_i[t] += (x[t] . A_i[s_t]^T) . B_i[s_t]^T * scaling, tokens grouped by slot.
//
// One launch over the work units of the two-launch form (sgmv.hip): the 64-token tiles of the long
// segments and, behind them in the same grid, the short segments.  A workgroup takes one (tile,
// column range): it multiplies the tile's x rows by A[slot] of the range's slice over the whole of
// K (the shrink of sgmv_body.h with its sums left in LDS), then expands the result into its column
// range (the expand of sgmv_body.h on an intermediate that is in LDS already).  Nothing passes
// between workgroups and nothing between launches: no workspace, no second launch with its
// launch-to-first-byte latency, and no K parts.  The price is that every column range of a tile
// repeats the tile's shrink: its x rows and the slot's A rows come from the XCD's L2 after the
// first range has fetched them (a tile's ranges are dispatched together on one XCD), so the
// repeats cost compute-unit intake, not HBM traffic.  The library takes this form where the
// repeats are few (wide_pays): projections of few, narrow slices over a short K.
#include "sgmv_body.h"

namespace mlora {

namespace {

template <typename T, int R, int KR, int XW, bool DB, int CPL, int TPF>
__global__ __launch_bounds__(kShrinkWaves* kWave, 2) void wide_kernel(const int32_t* __restrict__ plan, const void* __restrict__ xv,
                                                                      void* __restrict__ yv_, int64_t xs, int64_t ys, int big_off, int small_off,
                                                                      int big_cap, int bigrows_off, int T_, int K, int num_slots, int num_slices,
                                                                      float scaling, const int32_t* __restrict__ eff_rank, ShrinkSlices sl,
                                                                      ExpandSplits splits) {
  static_assert(kShrinkWaves == kExpandWaves, "one workgroup runs both bodies");
  constexpr int ASTRIDE = KR + 8;
  constexpr int HSTRIDE = 2 * R + 8;
  constexpr int A_ELEMS = R * ASTRIDE, H_ELEMS = MLORA_TILE_BIG * HSTRIDE;
  // the A slabs of the shrink and, once it is over, the intermediate of the expand
  __shared__ __attribute__((aligned(16))) T s_raw[A_ELEMS > H_ELEMS ? A_ELEMS : H_ELEMS];
  __shared__ __attribute__((aligned(16))) int s_row[MLORA_TILE_BIG];
  __shared__ int s_slot[1], s_m[1], s_eff[1];

  const int tid = threadIdx.x;
  const int tile = tile_position(big_cap);  // blockIdx.x is the XCD
  MLORA_STAMP(0);  // first instruction
  // the token rows, requested with the record (their place follows from the tile's): the row of
  // this lane's position in the shrink, and (threads 0..63) of position tid for the expand
  const int row = tile_row(plan, bigrows_off, small_off, big_cap, tile, (tid / kWave) * 16 + (tid & 15));
  const int rowv1 = tid < MLORA_TILE_BIG ? tile_row(plan, bigrows_off, small_off, big_cap, tile, tid) : 0;
  const TileRef tr = fetch_tile(plan, big_off, small_off, big_cap, tile, T_, num_slots);
  const ExpandSplit sp = splits.split[blockIdx.y];
  if (!tr.ok || sp.n0 >= sp.n1) {
    count_rejected_plan(plan, tr.plan_ok);
    return;
  }
  MLORA_STAMP(1);  // tile record here
  // rank of the adapter in this slot (a second, dependent fetch, only with the vector given)
  int eff = R;
  if (eff_rank) {
    eff = eff_rank[tr.slot];
    eff = eff < 0 ? 0 : eff > R ? R : eff;
    if (eff == 0) return;
  }
  const int slot[1] = {tr.slot}, start[1] = {tr.start}, m[1] = {tr.m}, effv[1] = {eff}, rowv[1] = {rowv1};
  if (eff < R) {
    if (R > 16 && ((eff + 15) >> 4) < (R + 15) / 16)
      shrink_body<T, R, KR, XW, DB, true, false, true>(s_raw, xv, nullptr, xs, T_, K, num_slices, K, 0, sl, sp.slice, 0, tr.slot, tr.start, tr.m, eff, row,
                                                       s_raw, scaling);
    else
      shrink_body<T, R, KR, XW, DB, false, false, true>(s_raw, xv, nullptr, xs, T_, K, num_slices, K, 0, sl, sp.slice, 0, tr.slot, tr.start, tr.m, eff,
                                                        row, s_raw, scaling);
    MLORA_STAMP(6);  // intermediate on its way to LDS
    expand_body<T, R, CPL, TPF, 1, true, false, true>(s_raw, s_row, s_slot, s_m, s_eff, plan, nullptr, yv_, ys, T_, num_slices, 1, scaling, sp, slot,
                                                      start, m, effv, rowv);
  } else {
    shrink_body<T, R, KR, XW, DB, false, false, true>(s_raw, xv, nullptr, xs, T_, K, num_slices, K, 0, sl, sp.slice, 0, tr.slot, tr.start, tr.m, eff, row,
                                                      s_raw, scaling);
    MLORA_STAMP(6);
    expand_body<T, R, CPL, TPF, 1, false, false, true>(s_raw, s_row, s_slot, s_m, s_eff, plan, nullptr, yv_, ys, T_, num_slices, 1, scaling, sp, slot,
                                                       start, m, effv, rowv);
  }
}

struct WideLaunch {
  const MloraAddArgs* a;
  PlanLayout lay;
  ShrinkSlices sl;
  ExpandSplits splits;
  dim3 grid;
  int big_cap;
};

template <typename T, int R, int KR>
void launch_wide_one(const WideLaunch& l) {
  const MloraAddArgs* a = l.a;
  hipLaunchKernelGGL((wide_kernel<T, R, KR, KR, true, 8, 2>), l.grid, dim3(kShrinkWaves * kWave), 0, static_cast<hipStream_t>(a->stream), a->plan,
                     a->x, a->y, a->x_stride, a->y_stride, l.lay.big_off, l.lay.small_off, l.big_cap, l.lay.bigrows_off, a->num_tokens, a->k,
                     a->num_slots, a->num_slices, a->scaling, a->effective_rank, l.sl, l.splits);
}

template <typename T>
void launch_wide_rank(const WideLaunch& l) {
  const bool k256 = l.a->k % 256 == 0;
  switch (l.a->r) {
    case 8: k256 ? launch_wide_one<T, 8, 256>(l) : launch_wide_one<T, 8, 128>(l); break;
    case 16: k256 ? launch_wide_one<T, 16, 256>(l) : launch_wide_one<T, 16, 128>(l); break;
    case 32: k256 ? launch_wide_one<T, 32, 256>(l) : launch_wide_one<T, 32, 128>(l); break;
    default: k256 ? launch_wide_one<T, 64, 256>(l) : launch_wide_one<T, 64, 128>(l); break;
  }
}

// Diagnostic knob, read from the environment once and again after mlora_reload_knobs().
struct WideKnobs {
  int generation = -1, nt;
  void read() {
    generation = knob_generation();
    nt = env_int("MLORA_WIDE_NT", 0);  // columns per range (0: 512)
  }
};
const WideKnobs& wide_knobs() {
  static WideKnobs k;
  if (k.generation != knob_generation()) k.read();
  return k;
}

}  // namespace

void wide_trace_set(void* buf) {
#ifdef MLORA_TRACE
  (void)hipMemcpyToSymbol(HIP_SYMBOL(trace_buf), &buf, sizeof(buf));
#else
  (void)buf;
#endif
}

// Whether this form beats the two-launch one.  What it saves is a launch with its latency from
// launch to first byte, and the partial sums' trip through the workspace; what it adds is the
// intake of x and A rows by every column range of a tile beyond the first of its slice.  Measured
// on the prefill and the mixed batch (us per call, this form / two launches): qkv (K = 1024, ranges
// beyond the slices' first: 1) 24.8 / 28.6 and 35.9 / 41.6; o (K = 1024, 1) 17.2 / 18.0 and 19.9 /
// 23.0; gate_up (K = 1024, 14) 92.0 / 67.6; down (K = 4096, 1) 38.8 / 31.1: taken while the repeats
// are at most 1024 columns of K per tile.
bool wide_pays(const MloraAddArgs* a) {
  long long repeats = 0;
  for (int i = 0; i < a->num_slices; ++i) repeats += (a->slices[i].n + 511) / 512 - 1;
  return repeats * a->k <= 1024;
}

bool wide_supported(const MloraAddArgs* a) {
  if (!(a->k % 128 == 0 && a->k >= 128 && exact_rank(a->r))) return false;
  for (int i = 0; i < a->num_slices; ++i)
    if (a->slices[i].n <= 0) return false;
  return true;
}

int launch_wide(const MloraAddArgs* a) {
  const SgmvShape sh = sgmv_shape(a);
  if (sh.empty) return 0;
  WideLaunch l;
  l.a = a; l.lay = sh.lay; l.sl = sh.sl; l.big_cap = sh.big_cap;
  // Column ranges of 512 columns (a span of 128 per wavefront).  Measured on the prefill batch (7608
  // tokens with adapter, rank 64; us per call at 512 / 1024 / 4096 columns): qkv 24.8 / 27.6 / 27.9,
  // o 17.2 / 21.2 / 21.4 (wider ranges leave compute units without a workgroup), gate_up 92.0 / 75.7 /
  // 68.2, down 38.8 / 43.5 / 43.6 (where the two-launch form is taken instead, wide_pays()).
  int nt = wide_knobs().nt;
  if (nt <= 0) nt = 512;
  const int nsplit = fill_splits(a, nt, l.splits.split);
  l.grid = dim3(8, static_cast<unsigned>(nsplit), static_cast<unsigned>(sh.tiles8));
  if (a->dtype == MLORA_DTYPE_BF16) launch_wide_rank<__bf16>(l);
  else launch_wide_rank<_Float16>(l);
  return check_launch("mlora_add_lora(64-token tiles, one launch)");
}

}  // namespace mlora
