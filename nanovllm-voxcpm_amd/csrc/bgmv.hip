// Vector-ALU alternative to decode.hip for the same computation (reference:
// nanovllm_voxcpm/lora.py:291-381, lora_ops/triton_ops/lora_shrink_op.py:104-210).
//
// BGMV form (vector ALU): one workgroup per (small tile, slice, column range).  A small tile is
// up to sixteen tokens that share a slot; the workgroup takes them eight at a time.
//   shrink  — every lane takes one 128-bit chunk of K, forms the partial dot products of its
//             tile rows with eight A rows (packed dot2, fp32 accumulate) and the 64 partials per
//             lane are folded across the wavefront with a halving butterfly (63 exchanges);
//   stage   — the rank-r intermediate lives in LDS only;
//   expand  — lanes read B as consecutive 128-bit chunks, r/8 lanes per output column, the
//             products are transposed through LDS and y is updated with 128-bit accesses.
#include "common.h"
#include "launch.h"

namespace mlora {

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;
constexpr int kMT = 8;  // tokens handled per pass over a small tile
constexpr int kColTile = 512;  // output columns staged in LDS at a time
constexpr int kMaxSplits = 64;

struct BgmvSplit {
  const void* a;
  const void* b;
  int n, y_col, n0, n1;
};

struct BgmvParams {
  const void* x;
  void* y;
  int64_t xs, ys;
  const int32_t* plan;
  int small_off;
  int T, K, num_slots, nsplit, include_long;
  float scaling;
  BgmvSplit split[kMaxSplits];
};

// Sum v[i] over the 64 lanes for all 64 i at once: at each step a lane hands the half it
// does not keep to its partner.  Afterwards lane l holds the total of v[l] in v[0].
template <int W>
__device__ __forceinline__ void wave_fold_step(float (&v)[64], int lane) {
  const bool up = (lane & W) != 0;
#pragma unroll
  for (int i = 0; i < W; ++i) {
    const float keep = up ? v[i + W] : v[i];
    const float send = up ? v[i] : v[i + W];
    v[i] = keep + __shfl_xor(send, W, kWave);
  }
}

__device__ __forceinline__ void wave_fold64(float (&v)[64], int lane) {
  wave_fold_step<32>(v, lane);
  wave_fold_step<16>(v, lane);
  wave_fold_step<8>(v, lane);
  wave_fold_step<4>(v, lane);
  wave_fold_step<2>(v, lane);
  wave_fold_step<1>(v, lane);
}

template <typename T, int R>
__global__ __launch_bounds__(kThreads) void bgmv_kernel(BgmvParams p) {
  constexpr int RG = R / 8;               // groups of eight A rows
  constexpr int WR = RG < kWaves ? RG : kWaves;  // waves spread over row groups ...
  constexpr int KS = kWaves / WR;         // ... and over K
  constexpr int LPC = R / 8;              // lanes per output column in the expand
  constexpr int DSTRIDE = kColTile + (LPC > 1 ? 64 / LPC : 0);

  __shared__ float s_part[KS * RG * 64];
  __shared__ float s_h[kMT * R];
  __shared__ float s_delta[kMT * DSTRIDE];
  __shared__ int s_row[kMT];

  // Workgroups b, b+8, b+16, ... share an XCD (and its L2): give them the column ranges of
  // one tile so that x rows and A[slot] are fetched into that L2 once.
  // grid (8, column ranges, tiles / 8): linear workgroup ids advance along x first, and
  // consecutive ids go to consecutive XCDs, so blockIdx.x is the XCD
  const int split_id = blockIdx.y;
  const int tile = blockIdx.z * 8 + blockIdx.x;
  const int32_t* hdr = p.plan;
  const int32_t* rec = p.plan + p.small_off + tile * MLORA_SMALL_TILE_WORDS;  // tile < capacity: in bounds
  const int slot = rec[0], m_tile = rec[1];
  if (hdr[MLORA_PLAN_MAGIC] != MLORA_PLAN_MAGIC_VALUE || hdr[MLORA_PLAN_NUM_TOKENS] != p.T ||
      hdr[MLORA_PLAN_MAX_SLOTS] != p.num_slots) {
    count_rejected_plan(p.plan, false);
    return;
  }
  const int n_tiles = hdr[MLORA_PLAN_TILES_SHORT] + (p.include_long ? hdr[MLORA_PLAN_TILES_LONG_SMALL] : 0);
  if (tile >= n_tiles) return;

  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  for (int part = 0; part * kMT < m_tile; ++part) {
  const int m = m_tile - part * kMT < kMT ? m_tile - part * kMT : kMT;
  const int32_t* sorted = rec + MLORA_SMALL_TILE_ROWS + part * kMT;
  int rows[kMT];
#pragma unroll
  for (int t = 0; t < kMT; ++t) rows[t] = sorted[t < m ? t : 0];
  if (tid < kMT) s_row[tid] = rows[0];
  if (tid < m) s_row[tid] = sorted[tid];

  const BgmvSplit sp = p.split[split_id];
  const T* x = static_cast<const T*>(p.x);
  const T* A = static_cast<const T*>(sp.a) + static_cast<int64_t>(slot) * R * p.K;
  const int K = p.K;

  // ---- shrink ---------------------------------------------------------------------------
  {
    const int wr = wave % WR, ks = wave / WR;
    const int KP = (K + 511) / 512;  // 512 elements of K per wavefront pass
    for (int rg = wr; rg < RG; rg += WR) {
      float acc[64];
#pragma unroll
      for (int i = 0; i < 64; ++i) acc[i] = 0.f;
      for (int kp = ks; kp < KP; kp += KS) {
        const int c = (kp * kWave + lane) * 8;
        if (c < K) {
          Pack8 xv[kMT];
#pragma unroll
          for (int t = 0; t < kMT; ++t)
            if (t < m) xv[t].raw = load128(x + static_cast<int64_t>(rows[t]) * p.xs + c);
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            Pack8 av;
            av.raw = load128(A + static_cast<int64_t>(rg * 8 + j) * K + c);
#pragma unroll
            for (int t = 0; t < kMT; ++t)
              if (t < m) acc[t * 8 + j] = dot8<T>(xv[t], av, acc[t * 8 + j]);
          }
        }
      }
      wave_fold64(acc, lane);
      s_part[(ks * RG + rg) * 64 + lane] = acc[0];
    }
  }
  __syncthreads();
  for (int e = tid; e < kMT * R; e += kThreads) {
    const int t = e / R, jj = e % R, rg = jj / 8, j = jj % 8;
    float sum = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) sum += s_part[(ks * RG + rg) * 64 + t * 8 + j];
    s_h[e] = sum * p.scaling;
  }
  __syncthreads();

  // ---- expand ---------------------------------------------------------------------------
  const int kq = tid % LPC;  // which eight ranks of a B row this lane multiplies
  float hreg[kMT][8];
#pragma unroll
  for (int t = 0; t < kMT; ++t)
#pragma unroll
    for (int e = 0; e < 8; ++e) hreg[t][e] = s_h[t * R + kq * 8 + e];

  const T* B = static_cast<const T*>(sp.b) + static_cast<int64_t>(slot) * sp.n * R;
  T* y = static_cast<T*>(p.y) + sp.y_col;
  for (int c0 = sp.n0; c0 < sp.n1; c0 += kColTile) {
    const int cend = c0 + kColTile < sp.n1 ? c0 + kColTile : sp.n1;
    for (int n = c0 + tid / LPC; n < cend; n += kThreads / LPC) {
      Pack8 bv;
      bv.raw = load128(B + static_cast<int64_t>(n) * R + kq * 8);
      float bf[8];
      unpack8<T>(bv, bf);
#pragma unroll
      for (int t = 0; t < kMT; ++t) {
        if (t < m) {
          float pt = 0.f;
#pragma unroll
          for (int e = 0; e < 8; ++e) pt += hreg[t][e] * bf[e];
#pragma unroll
          for (int o = 1; o < LPC; o <<= 1) pt += __shfl_xor(pt, o, kWave);
          if ((t % LPC) == kq) s_delta[t * DSTRIDE + (n - c0)] = pt;
        }
      }
    }
    __syncthreads();
    const int chunks = (cend - c0) >> 3;
    for (int cid = tid; cid < m * chunks; cid += kThreads) {
      const int t = cid / chunks, c8 = cid - t * chunks;
      T* yp = y + static_cast<int64_t>(s_row[t]) * p.ys + c0 + c8 * 8;
      Pack8 yv;
      yv.raw = load128(yp);
      float yf[8];
      unpack8<T>(yv, yf);
      const float* d = s_delta + t * DSTRIDE + c8 * 8;
#pragma unroll
      for (int e = 0; e < 8; ++e) yf[e] += d[e];
      pack8<T>(yf, yv);
      store128(yp, yv.raw);
    }
    __syncthreads();
  }
  }  // next eight tokens of the tile
}

template <typename T>
void launch_rank(const BgmvParams& p, int r, dim3 grid, hipStream_t st) {
  switch (r) {
    case 8: hipLaunchKernelGGL((bgmv_kernel<T, 8>), grid, dim3(kThreads), 0, st, p); break;
    case 16: hipLaunchKernelGGL((bgmv_kernel<T, 16>), grid, dim3(kThreads), 0, st, p); break;
    case 32: hipLaunchKernelGGL((bgmv_kernel<T, 32>), grid, dim3(kThreads), 0, st, p); break;
    default: hipLaunchKernelGGL((bgmv_kernel<T, 64>), grid, dim3(kThreads), 0, st, p); break;
  }
}

}  // namespace

int launch_bgmv(const MloraAddArgs* a, bool include_long) {
  BgmvParams p;
  p.x = a->x; p.y = a->y; p.xs = a->x_stride; p.ys = a->y_stride;
  p.plan = a->plan;
  const PlanLayout lay = plan_layout(a->num_tokens, a->num_slots);
  p.small_off = lay.small_off;
  p.T = a->num_tokens; p.K = a->k; p.num_slots = a->num_slots; p.include_long = include_long ? 1 : 0;
  p.scaling = a->scaling;

  // Column ranges: about `nt` columns per workgroup, widened until the table fits.
  int nt = env_int("MLORA_BGMV_NT", 512);
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
  for (int i = 0; i < a->num_slices; ++i) {
    const MloraSlice& sl = a->slices[i];
    for (int n0 = 0; n0 < sl.n; n0 += nt) {
      BgmvSplit& sp = p.split[s++];
      sp.a = sl.a; sp.b = sl.b; sp.n = sl.n; sp.y_col = sl.y_col;
      sp.n0 = n0; sp.n1 = n0 + nt < sl.n ? n0 + nt : sl.n;
    }
  }
  p.nsplit = total;

  int cap = lay.cap_small;
  if (!include_long) {
    const int segs = a->num_slots < a->num_tokens ? a->num_slots : a->num_tokens;
    if (segs < cap) cap = segs;  // a segment below the threshold is exactly one small tile
  }
  if (cap == 0) return 0;
  cap = (cap + 7) & ~7;
  dim3 grid(8, static_cast<unsigned>(total), static_cast<unsigned>(cap / 8));
  hipStream_t st = static_cast<hipStream_t>(a->stream);
  if (a->dtype == MLORA_DTYPE_BF16) launch_rank<__bf16>(p, a->r, grid, st);
  else launch_rank<_Float16>(p, a->r, grid, st);
  return check_launch("mlora_add_lora(bgmv)");
}

}  // namespace mlora
