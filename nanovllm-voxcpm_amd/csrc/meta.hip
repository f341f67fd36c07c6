// On-device segment metadata: a stable counting sort of the tokens by slot id, run by one
// workgroup, that emits (a) the plan workspace the apply kernels walk and (b) any of the
// three index layouts the reference builds on the host: the engine's (slots ascending, -1
// left out: nanovllm_voxcpm/engine/lora_manager.py:77-91, utils/context.py:77-116), the kernel
// metadata's (-1 bucket first: lora_ops/triton_ops/lora_kernel_metadata.py:46-68) and the graph
// buffers' (fixed ids -1 .. L-1, counts scattered: engine/model_runner.py:727-797).
#include "common.h"

namespace mlora {

namespace {

constexpr int kMetaThreads = 512;
constexpr int kMetaWaves = kMetaThreads / kWave;

struct MetaParams {
  const int32_t* tts;
  int T, L, no_lora_bucket;
  int32_t* plan;
  int32_t* sorted_idx;
  int32_t* compact_ids;
  int32_t* compact_counts;
  int32_t* compact_offsets;
  int compact_capacity;
  int32_t* dense_counts;
  int32_t* dense_offsets;
  int32_t* padded_tts;
  int padded_len;
  int32_t* scalars;
};

__device__ __forceinline__ int wave_incl_scan(int v, int lane) {
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    int n = __shfl_up(v, o, kWave);
    if (lane >= o) v += n;
  }
  return v;
}

// Largest b in [0, n) with arr[b] <= q, for a non-decreasing arr[0..n].
__device__ __forceinline__ int find_bucket(const int* arr, int n, int q) {
  int lo = 0, hi = n;  // invariant: arr[lo] <= q < arr[hi]
  while (hi - lo > 1) {
    int mid = (lo + hi) >> 1;
    if (arr[mid] <= q) lo = mid; else hi = mid;
  }
  return lo;
}

__global__ __launch_bounds__(kMetaThreads) void meta_kernel(MetaParams p) {
  extern __shared__ int lds[];
  const int NB = p.L + 1;  // bucket b holds slot b - 1; bucket 0 is "no LoRA"
  int* hist = lds;                     // [waves][NB]: per-wave counts, later running write cursors
  int* total = hist + kMetaWaves * NB; // [NB]
  int* off = total + NB;               // [NB + 1]: first position of bucket b among LoRA tokens
  int* cidx = off + NB + 1;            // [NB + 1]: compact index of bucket b
  int* ts_short = cidx + NB + 1;       // [NB + 1]: first small tile of a short segment
  int* ts_long = ts_short + NB + 1;    // [NB + 1]: first small tile of a long segment
  int* ts_big = ts_long + NB + 1;      // [NB + 1]: first big tile of a long segment
  int* ts_over = ts_big + NB + 1;      // [NB + 1]: first of the small tiles behind a slot's first one
  __shared__ int s_bad, s_max;
  __shared__ int s_nlong;              // slots with a long segment

  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int T = p.T, L = p.L;

  for (int i = tid; i < kMetaWaves * NB; i += kMetaThreads) hist[i] = 0;
  if (tid == 0) { s_bad = 0; s_max = 0; }
  __syncthreads();

  // Each wave owns one contiguous span of tokens, so wave order equals token order.
  int span = (T + kMetaWaves - 1) / kMetaWaves;
  span = (span + kWave - 1) & ~(kWave - 1);
  const int beg = wave * span;
  const int end = beg + span < T ? beg + span : T;

  // A wavefront walks its span in steps of 64 tokens with the slot ids of the next four steps
  // requested ahead: a step is a few hundred cycles of work and a request to memory takes several
  // times that, so with one step in flight the walk runs at the pace of the memory's latency.
  constexpr int kAhead = 4;
  auto walk = [&](auto&& step) {
    int q[kAhead];
#pragma unroll
    for (int j = 0; j < kAhead; ++j) {
      const int t = beg + j * kWave + lane;
      q[j] = t < end ? p.tts[t] : -1;
    }
    for (int base = beg; base < end; base += kAhead * kWave) {
#pragma unroll
      for (int j = 0; j < kAhead; ++j) {
        const int t = base + j * kWave + lane;
        const int s = q[j];
        const int tn = t + kAhead * kWave;
        q[j] = tn < end ? p.tts[tn] : -1;
        if (base + j * kWave < end) step(t, s);
      }
    }
  };
  walk([&](int t, int s) {
    if (t < end) {
      int key = (s >= 0 && s < L) ? s + 1 : 0;
      if (s >= L) s_bad = 1;
      atomicAdd(&hist[wave * NB + key], 1);
    }
  });
  if (p.padded_tts) {
    for (int i = tid; i < p.padded_len; i += kMetaThreads) p.padded_tts[i] = i < T ? p.tts[i] : -1;
  }
  __syncthreads();

  // Per bucket: turn the per-wave counts into exclusive prefixes over waves.
  for (int b = tid; b < NB; b += kMetaThreads) {
    int run = 0;
    for (int w = 0; w < kMetaWaves; ++w) {
      int c = hist[w * NB + b];
      hist[w * NB + b] = run;
      run += c;
    }
    total[b] = run;
  }
  __syncthreads();

  // Wave 0: exclusive scans over the buckets.
  const int b0 = p.no_lora_bucket ? 0 : 1;  // first bucket of the compact arrays
  if (wave == 0) {
    int run0 = 0, run1 = 0, run2 = 0, run3 = 0, run4 = 0, run5 = 0, mx = 0, nlong = 0;
    for (int base = 0; base < NB; base += kWave) {
      int b = base + lane;
      int c_all = b < NB ? total[b] : 0;
      int c = b >= 1 ? c_all : 0;  // LoRA tokens only
      bool is_short = c < MLORA_SEGMENT_THRESHOLD;
      int v0 = c;
      int v1 = (b >= b0 && c_all > 0) ? 1 : 0;
      int nsmall = (c + MLORA_TILE_SMALL - 1) / MLORA_TILE_SMALL;
      int v2 = is_short ? nsmall : 0;
      int v3 = is_short ? 0 : nsmall;
      int v4 = is_short ? 0 : (c + MLORA_TILE_BIG - 1) / MLORA_TILE_BIG;
      int v5 = nsmall > 1 ? nsmall - 1 : 0;
      int i0 = wave_incl_scan(v0, lane), i1 = wave_incl_scan(v1, lane), i2 = wave_incl_scan(v2, lane);
      int i3 = wave_incl_scan(v3, lane), i4 = wave_incl_scan(v4, lane), i5 = wave_incl_scan(v5, lane);
      if (b < NB) {
        off[b] = run0 + i0 - v0;
        cidx[b] = run1 + i1 - v1;
        ts_short[b] = run2 + i2 - v2;
        ts_long[b] = run3 + i3 - v3;
        ts_big[b] = run4 + i4 - v4;
        ts_over[b] = run5 + i5 - v5;
      }
      run0 += __shfl(i0, kWave - 1, kWave);
      run1 += __shfl(i1, kWave - 1, kWave);
      run2 += __shfl(i2, kWave - 1, kWave);
      run3 += __shfl(i3, kWave - 1, kWave);
      run4 += __shfl(i4, kWave - 1, kWave);
      run5 += __shfl(i5, kWave - 1, kWave);
      nlong += __popcll(__ballot(b < NB && !is_short));
      int m = c;
#pragma unroll
      for (int o = 32; o >= 1; o >>= 1) { int n = __shfl_xor(m, o, kWave); m = n > m ? n : m; }
      mx = m > mx ? m : mx;
    }
    if (lane == 0) {
      off[NB] = run0; cidx[NB] = run1; ts_short[NB] = run2; ts_long[NB] = run3; ts_big[NB] = run4; ts_over[NB] = run5;
      s_max = mx;
      s_nlong = nlong;
    }
  }
  __syncthreads();

  const int n_lora = off[NB];
  // With the "no LoRA" bucket requested and no LoRA token at all, the reference's builder returns
  // early and leaves its buffers in the reset state (ids -1, counts 0, offsets 0, sort untouched).
  const bool reset_only = p.no_lora_bucket && n_lora == 0;
  const int n_neg = (p.no_lora_bucket && !reset_only) ? total[0] : 0;  // tokens sorted ahead of every slot
  const int n_compact = reset_only ? 0 : cidx[NB];
  const int n_short = ts_short[NB], n_long = ts_long[NB], n_big = ts_big[NB], n_over = ts_over[NB];
  const PlanLayout lay = plan_layout(T, L);

  if (tid == 0) {
    if (p.plan) {
      int32_t* h = p.plan;
      h[MLORA_PLAN_MAGIC] = MLORA_PLAN_MAGIC_VALUE;
      h[MLORA_PLAN_NUM_TOKENS] = T;
      h[MLORA_PLAN_MAX_SLOTS] = L;
      h[MLORA_PLAN_NUM_LORA_TOKENS] = n_lora;
      h[MLORA_PLAN_NUM_ACTIVE] = cidx[NB] - ((p.no_lora_bucket && total[0] > 0) ? 1 : 0);
      h[MLORA_PLAN_NO_LORA] = n_lora == 0;
      h[MLORA_PLAN_BAD_SLOT] = s_bad;
      h[MLORA_PLAN_TILES_SHORT] = n_short;
      h[MLORA_PLAN_TILES_LONG_SMALL] = n_long;
      h[MLORA_PLAN_TILES_LONG_BIG] = n_big;
      h[MLORA_PLAN_MAX_SEGMENT] = s_max;
      h[MLORA_PLAN_TILES_OVER] = n_over;
      for (int i = MLORA_PLAN_TILES_OVER + 1; i < MLORA_PLAN_HEADER_WORDS; ++i) h[i] = 0;  // (MLORA_PLAN_REJECTED among them)
    }
    if (p.scalars) {
      p.scalars[0] = n_compact;
      p.scalars[1] = n_lora + n_neg;
      p.scalars[2] = n_lora == 0;
      p.scalars[3] = s_bad;
    }
    if (p.dense_offsets) p.dense_offsets[0] = 0;
    if (p.compact_offsets) p.compact_offsets[n_compact] = n_lora + n_neg;
    if (p.plan) p.plan[lay.offsets_off] = 0;
  }

  // Per-bucket outputs.
  for (int b = tid; b < NB; b += kMetaThreads) {
    const int c = b >= 1 ? total[b] : 0;
    if (p.dense_counts) p.dense_counts[b] = c;
    if (p.dense_offsets) p.dense_offsets[b + 1] = off[b + 1];
    if (p.plan) {
      p.plan[lay.counts_off + b] = c;
      p.plan[lay.offsets_off + b + 1] = off[b + 1];
    }
    const int c_all = total[b];
    if (!reset_only && b >= b0 && c_all > 0) {
      const int i = cidx[b];
      if (p.compact_ids) p.compact_ids[i] = b - 1;
      if (p.compact_counts) p.compact_counts[i] = c_all;
      if (p.compact_offsets) p.compact_offsets[i] = b == 0 ? 0 : n_neg + off[b];
    }
  }
  for (int i = n_compact + tid; i < p.compact_capacity; i += kMetaThreads) {
    if (p.compact_ids) p.compact_ids[i] = -1;
    if (p.compact_counts) p.compact_counts[i] = 0;
    if (p.compact_offsets) p.compact_offsets[i + 1] = 0;
  }

  // Tile lists of the plan.  A small-tile record starts with its header and zeroed row entries;
  // the scatter below fills all sixteen (the tile's tokens, repeated cyclically past its count).
  i32x4* small = p.plan ? reinterpret_cast<i32x4*>(p.plan + lay.small_off) : nullptr;
  // place of big tile q (in slot order) in the list: runs of `run` consecutive tiles go to the
  // blocks (XCDs) in turn
  const int run = big_tile_run(n_big, s_nlong);
  auto place_big = [&](int q) { return big_tile_place(q, run, lay.cap_big); };
  if (p.plan) {
    i32x4* big = reinterpret_cast<i32x4*>(p.plan + lay.big_off);
    for (int q = tid; q < lay.cap_big; q += kMetaThreads) big[q] = i32x4{-1, 0, 0, 0};
    __syncthreads();  // (a place is cleared by one thread and may be filled by another)
    for (int q = tid; q < n_short + n_long; q += kMetaThreads) {
      const bool is_short = q < n_short;
      const int* ts = is_short ? ts_short : ts_long;
      const int qq = is_short ? q : q - n_short;
      const int b = find_bucket(ts, NB, qq);
      const int j = qq - ts[b], c = total[b];
      const int left = c - j * MLORA_TILE_SMALL;
      i32x4* rec = small + q * (MLORA_SMALL_TILE_WORDS / 4);
      rec[0] = i32x4{b - 1, left < MLORA_TILE_SMALL ? left : MLORA_TILE_SMALL, off[b] + j * MLORA_TILE_SMALL, 0};
#pragma unroll
      for (int w = 1; w < MLORA_SMALL_TILE_WORDS / 4; ++w) rec[w] = i32x4{0, 0, 0, 0};
    }
    for (int q = tid; q < n_big; q += kMetaThreads) {
      int b = find_bucket(ts_big, NB, q);
      int j = q - ts_big[b], c = total[b];
      int left = c - j * MLORA_TILE_BIG;
      big[place_big(q)] = i32x4{b - 1, off[b] + j * MLORA_TILE_BIG, left < MLORA_TILE_BIG ? left : MLORA_TILE_BIG, 0};
    }
    // row lists of the big tiles: cleared, the scatter below enters the tokens
    i32x4* rows = reinterpret_cast<i32x4*>(p.plan + lay.bigrows_off);
    for (int q = tid; q < n_big * (MLORA_TILE_BIG / 4); q += kMetaThreads)
      rows[place_big(q / (MLORA_TILE_BIG / 4)) * (MLORA_TILE_BIG / 4) + q % (MLORA_TILE_BIG / 4)] = i32x4{0, 0, 0, 0};
    // the small tiles once more, by slot: the record of every slot id (count 0 for a slot without
    // tokens and for the ids that round the list up to a multiple of eight), then the further
    // tiles of every slot, then count 0 up to the capacity
    const int check = static_cast<int>(MLORA_PLAN_CHECK(T, L));
    i32x4* byslot = reinterpret_cast<i32x4*>(p.plan + lay.slotrec_off);
    for (int q = tid; q < lay.cap_slotrec + lay.cap_over; q += kMetaThreads) {
      i32x4 head = i32x4{-1, 0, 0, check};
      if (q < L) {
        const int c = total[q + 1];
        head = i32x4{q, c < MLORA_TILE_SMALL ? c : MLORA_TILE_SMALL, off[q + 1], check};
      } else if (q >= lay.cap_slotrec && q - lay.cap_slotrec < n_over) {
        const int qq = q - lay.cap_slotrec;
        const int b = find_bucket(ts_over, NB, qq);
        const int j = qq - ts_over[b] + 1, left = total[b] - j * MLORA_TILE_SMALL;
        head = i32x4{b - 1, left < MLORA_TILE_SMALL ? left : MLORA_TILE_SMALL, off[b] + j * MLORA_TILE_SMALL, check};
      }
      i32x4* rec = byslot + q * (MLORA_SMALL_TILE_WORDS / 4);
      rec[0] = head;
#pragma unroll
      for (int w = 1; w < MLORA_SMALL_TILE_WORDS / 4; ++w) rec[w] = i32x4{0, 0, 0, 0};
    }
  }
  __syncthreads();

  // Stable scatter: every wave walks its span again in token order.  The rank of a token
  // among the equal keys of its 64-token step is counted lane against lane; the running cursor
  // of (wave, key) lives in hist and is advanced once per distinct key per step.
  int32_t* plan_sorted = p.plan ? p.plan + lay.sorted_off : nullptr;
  const uint64_t lt_mask = (lane == 0) ? 0ull : (~0ull >> (kWave - lane));
  const int key_bits = 32 - __builtin_clz(NB);  // keys are 0 .. NB - 1
  walk([&](int t, int s) {
    int key = -1;
    if (t < end) key = (s >= 0 && s < L) ? s + 1 : 0;
    const bool take = key >= 1 || (key == 0 && p.no_lora_bucket && !reset_only);
    // Rank of this token among the equal keys of its 64-token step, and the size of that group:
    // the set of lanes holding the same key is narrowed down one key bit at a time with ballots
    // (a fixed handful of steps, however many distinct keys the step holds).
    uint64_t peers = __ballot(take);
    for (int bit = 0; bit < key_bits; ++bit) {
      const uint64_t set = __ballot((key >> bit) & 1);
      peers &= ((key >> bit) & 1) ? set : ~set;
    }
    const int before = __popcll(peers & lt_mask), group = __popcll(peers);
    if (take) {
      const int cursor = hist[wave * NB + key];
      const int r = cursor + before;
      if (key >= 1) {
        if (plan_sorted) {
          plan_sorted[off[key] + r] = t;
          const int c = total[key];
          const int q = (c < MLORA_SEGMENT_THRESHOLD ? ts_short[key] : n_short + ts_long[key]) + r / MLORA_TILE_SMALL;
          // the token's own entry, and every entry past the tile's count that repeats it: a tile of
          // n < 16 tokens lists them cyclically, so that a kernel which fetches all sixteen rows
          // touches no memory beyond the rows of the tile itself
          const int tile = r / MLORA_TILE_SMALL;
          const int left = c - tile * MLORA_TILE_SMALL;
          const int n = left < MLORA_TILE_SMALL ? left : MLORA_TILE_SMALL;
          // (the same sixteen entries in the tile's record of the list by slot)
          const int q2 = tile == 0 ? key - 1 : lay.cap_slotrec + ts_over[key] + tile - 1;
          for (int pos = r % MLORA_TILE_SMALL; pos < MLORA_TILE_SMALL; pos += n) {
            p.plan[lay.small_off + q * MLORA_SMALL_TILE_WORDS + MLORA_SMALL_TILE_ROWS + pos] = t;
            p.plan[lay.slotrec_off + q2 * MLORA_SMALL_TILE_WORDS + MLORA_SMALL_TILE_ROWS + pos] = t;
          }
          // its entry in the row list of the segment's 64-token tile (entries past a tile's count
          // stay 0, a valid row: only the last tile of a segment has any, and repeating its tokens
          // there as in the small records is a loop of up to 64 stores in one lane)
          if (c >= MLORA_SEGMENT_THRESHOLD)
            p.plan[lay.bigrows_off + place_big(ts_big[key] + r / MLORA_TILE_BIG) * MLORA_TILE_BIG + r % MLORA_TILE_BIG] = t;
        }
        if (p.sorted_idx) p.sorted_idx[n_neg + off[key] + r] = t;
      } else if (p.sorted_idx) {
        p.sorted_idx[r] = t;
      }
      // the last lane of a group moves the group's cursor on (one writer per key; the wavefront's
      // LDS accesses execute in order, so the next step reads the new value)
      if (before == group - 1) hist[wave * NB + key] = cursor + group;
    }
    __builtin_amdgcn_wave_barrier();
  });
}

}  // namespace

}  // namespace mlora

using namespace mlora;

extern "C" size_t mlora_plan_workspace_bytes(int32_t num_tokens, int32_t max_slots) {
  if (num_tokens < 0 || max_slots < 0) return 0;
  return static_cast<size_t>(plan_layout(num_tokens, max_slots).total_words) * sizeof(int32_t);
}

extern "C" int mlora_meta_build(const MloraMetaArgs* a) {
  if (!a) { set_error("mlora_meta_build: NULL args"); return MLORA_E_INVALID; }
  if (a->num_tokens < 0 || a->max_slots < 0 || a->compact_capacity < 0 || a->padded_len < 0) {
    set_error("mlora_meta_build: negative size"); return MLORA_E_INVALID;
  }
  if (a->max_slots > MLORA_MAX_SLOTS) {
    set_error("mlora_meta_build: max_slots=%d exceeds %d", a->max_slots, MLORA_MAX_SLOTS); return MLORA_E_TOO_LARGE;
  }
  if (a->num_tokens > 0 && !a->token_to_slot) { set_error("mlora_meta_build: NULL token_to_slot"); return MLORA_E_INVALID; }
  if (reinterpret_cast<uintptr_t>(a->plan) & 15) { set_error("mlora_meta_build: plan must be 16-byte aligned"); return MLORA_E_INVALID; }
  if (a->padded_token_to_slot && a->padded_len < a->num_tokens) {
    set_error("mlora_meta_build: padded_len=%d is shorter than num_tokens=%d", a->padded_len, a->num_tokens);
    return MLORA_E_INVALID;
  }
  const bool wants_compact = a->compact_ids || a->compact_counts || a->compact_offsets;
  if (wants_compact) {
    const int t = a->num_tokens, l = a->max_slots + (a->no_lora_bucket ? 1 : 0);
    const int need = t < l ? t : l;
    if (a->compact_capacity < need) {
      set_error("mlora_meta_build: compact_capacity=%d cannot hold %d buckets", a->compact_capacity, need);
      return MLORA_E_INVALID;
    }
  }
  MetaParams p;
  p.tts = a->token_to_slot; p.T = a->num_tokens; p.L = a->max_slots; p.no_lora_bucket = a->no_lora_bucket ? 1 : 0;
  p.plan = a->plan; p.sorted_idx = a->sorted_idx;
  p.compact_ids = a->compact_ids; p.compact_counts = a->compact_counts; p.compact_offsets = a->compact_offsets;
  p.compact_capacity = wants_compact ? a->compact_capacity : 0;
  p.dense_counts = a->dense_counts; p.dense_offsets = a->dense_offsets;
  p.padded_tts = a->padded_token_to_slot; p.padded_len = a->padded_len;
  p.scalars = a->scalars;
  const int NB = p.L + 1;
  const size_t lds = sizeof(int) * (static_cast<size_t>(kMetaWaves + 1) * NB + 6 * (NB + 1));
  hipLaunchKernelGGL(meta_kernel, dim3(1), dim3(kMetaThreads), lds, static_cast<hipStream_t>(a->stream), p);
  return check_launch("mlora_meta_build");
}
