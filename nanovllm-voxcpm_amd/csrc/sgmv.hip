// SGMV form: one workgroup per (segment tile, slice, column range), both products on the
// matrix cores (v_mfma_f32_16x16x32 bf16 / f16, fp32 accumulate).
//   shrink  — H[tokens x r] = X_tile . A[slot]^T.  The four wavefronts split K; every lane
//             feeds the MFMA straight from 128-bit global loads of x rows and A rows, so
//             neither operand is read twice by a workgroup.  The four partial tiles are
//             summed through LDS and the rank-r intermediate is kept there as a hi + lo pair of
//             operand-precision values (about 16 significant bits), so the expand loses nothing
//             that would show after the final rounding of y.
//   expand  — OUT^T[cols x tokens] = B[slot] . H^T.  The B rows fed to the four MFMAs of a
//             64-column span are interleaved (row rho of MFMA j is column 16*(rho/4) + 4j + rho%4)
//             so that a lane ends up with 16 consecutive output columns of one token: y is
//             read, accumulated and written with 128-bit accesses, a full 128-byte line per
//             token per quarter-wave, with no transposition pass.
#include "common.h"
#include "launch.h"

namespace mlora {

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;
constexpr int kMaxSplits = 64;

template <typename T> struct Mma;
template <> struct Mma<__bf16> {
  static __device__ __forceinline__ f32x4 run(const Pack8& a, const Pack8& b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.bf, b.bf, c, 0, 0, 0);
  }
};
template <> struct Mma<_Float16> {
  static __device__ __forceinline__ f32x4 run(const Pack8& a, const Pack8& b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a.hf, b.hf, c, 0, 0, 0);
  }
};

struct SgmvSplit {
  const void* a;
  const void* b;
  int n, y_col, n0, n1;
};

struct SgmvParams {
  const void* x;
  void* y;
  int64_t xs, ys;
  const int32_t* plan;
  int sorted_off, tiles_off, count_word;
  int T, K, num_slots, nsplit;
  float scaling;
  SgmvSplit split[kMaxSplits];
};

template <typename T, int R, int MTB>
__global__ __launch_bounds__(kThreads) void sgmv_kernel(SgmvParams p) {
  constexpr int TB = MTB / 16;                  // 16-token blocks per tile
  constexpr int RB = (R + 15) / 16;             // 16-rank blocks
  constexpr int KSTEPS = (R + 31) / 32;         // MFMA k-steps of the expand
  constexpr int HSTRIDE = R + 8;                // padded LDS row of the intermediate

  __shared__ __attribute__((aligned(16))) float s_red[kWaves * RB * 64 * 4];
  __shared__ __attribute__((aligned(16))) T s_hb[MTB * HSTRIDE];  // leading part of H
  __shared__ __attribute__((aligned(16))) T s_hl[MTB * HSTRIDE];  // remainder H - hi

  // grid (8, column ranges, tiles / 8): linear workgroup ids advance along x first, and
  // consecutive ids go to consecutive XCDs, so blockIdx.x is the XCD
  const int split_id = blockIdx.y;
  const int tile = blockIdx.z * 8 + blockIdx.x;
  // header and tile record are fetched together (the record address is in bounds for every
  // workgroup of the grid, whether or not the tile exists)
  const int32_t* hdr = p.plan;
  const i32x4 td = reinterpret_cast<const i32x4*>(p.plan + p.tiles_off)[tile];
  const int magic = hdr[MLORA_PLAN_MAGIC], plan_t = hdr[MLORA_PLAN_NUM_TOKENS], plan_l = hdr[MLORA_PLAN_MAX_SLOTS];
  const int n_tiles = hdr[p.count_word];
  if (magic != MLORA_PLAN_MAGIC_VALUE || plan_t != p.T || plan_l != p.num_slots || tile >= n_tiles) return;
  const int slot = td[0], start = td[1], m = td[2];

  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int lr = lane & 15, lg = lane >> 4;
  const int32_t* sorted = p.plan + p.sorted_off + start;
  const SgmvSplit sp = p.split[split_id];
  const int K = p.K;

  // Token row of this lane in each 16-token block (rows past the tile repeat its first row:
  // they feed the MFMA harmlessly and are never written back).
  int row[TB];
#pragma unroll
  for (int tb = 0; tb < TB; ++tb) {
    const int ti = tb * 16 + lr;
    row[tb] = sorted[ti < m ? ti : 0];
  }

  // ---- shrink ---------------------------------------------------------------------------
  {
    const T* x = static_cast<const T*>(p.x);
    const T* A = static_cast<const T*>(sp.a) + static_cast<int64_t>(slot) * R * K;
    const T* xptr[TB];
    const T* aptr[RB];
#pragma unroll
    for (int tb = 0; tb < TB; ++tb) xptr[tb] = x + static_cast<int64_t>(row[tb]) * p.xs + lg * 8;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const int rr = rb * 16 + lr;
      aptr[rb] = A + static_cast<int64_t>(rr < R ? rr : R - 1) * K + lg * 8;
    }
    f32x4 acc[TB][RB];
#pragma unroll
    for (int tb = 0; tb < TB; ++tb)
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) acc[tb][rb] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int nks = K / 32;
    const int ks0 = wave * nks / kWaves, ks1 = (wave + 1) * nks / kWaves;
    for (int ks = ks0; ks < ks1; ++ks) {
      Pack8 xa[TB], aw[RB];
#pragma unroll
      for (int tb = 0; tb < TB; ++tb)
        if (tb * 16 < m) xa[tb].raw = load128(xptr[tb] + ks * 32);
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) aw[rb].raw = load128(aptr[rb] + ks * 32);
#pragma unroll
      for (int tb = 0; tb < TB; ++tb)
        if (tb * 16 < m) {
#pragma unroll
          for (int rb = 0; rb < RB; ++rb) acc[tb][rb] = Mma<T>::run(xa[tb], aw[rb], acc[tb][rb]);
        }
    }

    // Sum the four K-partials one 16-token block at a time and keep the result in LDS at the
    // operand precision.  D layout: lane holds H[token 4*(lane/16)+i][rank lane%16].
#pragma unroll
    for (int tb = 0; tb < TB; ++tb) {
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
        *reinterpret_cast<f32x4*>(&s_red[((wave * RB + rb) * 64 + lane) * 4]) = acc[tb][rb];
      __syncthreads();
      const int ln = tid >> 2, i = tid & 3;
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) sum += s_red[((w * RB + rb) * 64 + ln) * 4 + i];
        const int tok = tb * 16 + 4 * (ln >> 4) + i, r = rb * 16 + (ln & 15);
        if (r < R) {
          const float v = sum * p.scaling;
          const T hi = from_f32<T>(v);
          s_hb[tok * HSTRIDE + r] = hi;
          s_hl[tok * HSTRIDE + r] = from_f32<T>(v - to_f32(hi));
        }
      }
      __syncthreads();
    }
  }

  // ---- expand ---------------------------------------------------------------------------
  Pack8 hop[TB][KSTEPS], hlo[TB][KSTEPS];
#pragma unroll
  for (int tb = 0; tb < TB; ++tb)
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      const int kc = lg + 4 * ks;
      if (kc * 8 < R) {
        hop[tb][ks].raw = load128(&s_hb[(tb * 16 + lr) * HSTRIDE + kc * 8]);
        hlo[tb][ks].raw = load128(&s_hl[(tb * 16 + lr) * HSTRIDE + kc * 8]);
      } else {
        hop[tb][ks].raw = i32x4{0, 0, 0, 0};
        hlo[tb][ks].raw = i32x4{0, 0, 0, 0};
      }
    }

  const T* B = static_cast<const T*>(sp.b) + static_cast<int64_t>(slot) * sp.n * R;
  T* y = static_cast<T*>(p.y) + sp.y_col;
  for (int c0 = sp.n0 + wave * 64; c0 < sp.n1; c0 += kWaves * 64) {
    Pack8 bop[4][KSTEPS];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int n = c0 + 16 * (lr >> 2) + 4 * j + (lr & 3);
      n = n < sp.n1 ? n : sp.n1 - 1;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        const int kc = lg + 4 * ks;
        if (kc * 8 < R) bop[j][ks].raw = load128(B + static_cast<int64_t>(n) * R + kc * 8);
        else bop[j][ks].raw = i32x4{0, 0, 0, 0};
      }
    }
#pragma unroll
    for (int tb = 0; tb < TB; ++tb) {
      if (tb * 16 >= m) continue;
      f32x4 acc[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
          acc[j] = Mma<T>::run(bop[j][ks], hlo[tb][ks], acc[j]);
          acc[j] = Mma<T>::run(bop[j][ks], hop[tb][ks], acc[j]);
        }
      }
      if (tb * 16 + lr < m) {
        T* yp = y + static_cast<int64_t>(row[tb]) * p.ys + c0 + 16 * lg;
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          if (c0 + 16 * lg + 8 * half < sp.n1) {
            Pack8 yv;
            yv.raw = load128(yp + 8 * half);
            float yf[8];
            unpack8<T>(yv, yf);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              yf[i] += acc[2 * half][i];
              yf[4 + i] += acc[2 * half + 1][i];
            }
            pack8<T>(yf, yv);
            store128(yp + 8 * half, yv.raw);
          }
        }
      }
    }
  }
}

template <typename T, int MTB>
void launch_rank(const SgmvParams& p, int r, dim3 grid, hipStream_t st) {
  switch (r) {
    case 8: hipLaunchKernelGGL((sgmv_kernel<T, 8, MTB>), grid, dim3(kThreads), 0, st, p); break;
    case 16: hipLaunchKernelGGL((sgmv_kernel<T, 16, MTB>), grid, dim3(kThreads), 0, st, p); break;
    case 32: hipLaunchKernelGGL((sgmv_kernel<T, 32, MTB>), grid, dim3(kThreads), 0, st, p); break;
    default: hipLaunchKernelGGL((sgmv_kernel<T, 64, MTB>), grid, dim3(kThreads), 0, st, p); break;
  }
}

// Column ranges of about `nt` columns (a multiple of 256: four wavefronts of 64 columns).
int fill_splits(const MloraAddArgs* a, int nt, SgmvSplit* out) {
  nt = (nt + 255) & ~255;
  if (nt < 256) nt = 256;
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
      SgmvSplit& sp = out[s++];
      sp.a = sl.a; sp.b = sl.b; sp.n = sl.n; sp.y_col = sl.y_col;
      sp.n0 = n0; sp.n1 = n0 + nt < sl.n ? n0 + nt : sl.n;
    }
  }
  return total;
}

}  // namespace

bool sgmv_supported(const MloraAddArgs* a) { return a->k % 32 == 0 && a->k >= 32; }

// 64-token tiles of the segments at or above the threshold.
int launch_sgmv(const MloraAddArgs* a) {
  SgmvParams p;
  p.x = a->x; p.y = a->y; p.xs = a->x_stride; p.ys = a->y_stride; p.plan = a->plan;
  const PlanLayout lay = plan_layout(a->num_tokens, a->num_slots);
  p.sorted_off = lay.sorted_off;
  p.T = a->num_tokens; p.K = a->k; p.num_slots = a->num_slots; p.scaling = a->scaling;
  p.tiles_off = lay.big_off; p.count_word = MLORA_PLAN_TILES_LONG_BIG;
  int cap = lay.cap_big;
  if (cap == 0) return 0;
  int cols = 0;
  for (int i = 0; i < a->num_slices; ++i) cols += a->slices[i].n;
  if (cols == 0) return 0;
  // Aim for a few workgroups per CU: tiles x column ranges of about 1024 workgroups.
  const int target = env_int("MLORA_SGMV_WGS", 1024);
  const int est_tiles = a->num_tokens / MLORA_TILE_BIG + 1;
  int nt = env_int("MLORA_SGMV_NT", 0);
  if (nt <= 0) {
    const long long want = static_cast<long long>(cols) * est_tiles / (target > 0 ? target : 1);
    nt = want > 8192 ? 8192 : static_cast<int>(want);
  }
  p.nsplit = fill_splits(a, nt, p.split);
  cap = (cap + 7) & ~7;
  dim3 grid(8, static_cast<unsigned>(p.nsplit), static_cast<unsigned>(cap / 8));
  hipStream_t st = static_cast<hipStream_t>(a->stream);
  if (a->dtype == MLORA_DTYPE_BF16) launch_rank<__bf16, MLORA_TILE_BIG>(p, a->r, grid, st);
  else launch_rank<_Float16, MLORA_TILE_BIG>(p, a->r, grid, st);
  return check_launch("mlora_add_lora(mfma, big tiles)");
}

}  // namespace mlora
