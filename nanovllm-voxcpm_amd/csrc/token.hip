// Shape- and dtype-agnostic kernels: one workgroup per token, scalar loads.  They carry the
// fp32 / odd-shape cases of the fused apply, the unfused shrink and expand of the low-level
// API, and the slot install.  Nothing here needs segment metadata: a token's slot id is all
// a workgroup reads.  Reference semantics followed: lora_shrink (zero-filled output, scaling in
// the shrink: lora_ops/triton_ops/lora_shrink_op.py:257-341), lora_expand (offset_start,
// add_inputs, product rounded to B's type first: lora_expand_op.py:94-170), set_slot_lora
// (slot zeroed, rank-limited copy, alpha / r folded into B: nanovllm_voxcpm/layers/lora.py:395-417).
#include "common.h"

namespace mlora {

namespace {

constexpr int kTokThreads = 256;
constexpr int kTokWaves = kTokThreads / kWave;

struct TokenAddParams {
  const void* x; void* y;
  int64_t xs, ys;
  const int32_t* tts;
  int T, K, r, num_slots, nsplit;
  float scaling;
  const int32_t* eff_rank;  // per slot, or null
  MloraSlice slices[MLORA_MAX_SLICES];
};

// y[t, cols of slice] += scaling * (x[t] . A[s]^T) . B[s]^T   for grid (token, column split, slice)
template <typename T>
__global__ __launch_bounds__(kTokThreads) void token_add_kernel(TokenAddParams p) {
  __shared__ float h[MLORA_MAX_RANK];
  const int t = blockIdx.x;
  const int s = p.tts[t];
  if (s < 0 || s >= p.num_slots) return;
  const MloraSlice sl = p.slices[blockIdx.z];
  const int chunk = (sl.n + p.nsplit - 1) / p.nsplit;
  const int n0 = blockIdx.y * chunk;
  const int n1 = n0 + chunk < sl.n ? n0 + chunk : sl.n;
  if (n0 >= n1) return;
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const T* x = static_cast<const T*>(p.x) + static_cast<int64_t>(t) * p.xs;
  const T* A = static_cast<const T*>(sl.a) + static_cast<int64_t>(s) * p.r * p.K;
  // rows of A and columns of B at or above the rank of the adapter in this slot are not read
  int eff = p.r;
  if (p.eff_rank) {
    eff = p.eff_rank[s];
    eff = eff < 0 ? 0 : eff > p.r ? p.r : eff;
    if (eff == 0) return;
  }
  for (int j = wave; j < eff; j += kTokWaves) {
    const T* a = A + static_cast<int64_t>(j) * p.K;
    float acc = 0.f;
    for (int k = lane; k < p.K; k += kWave) acc += to_f32(x[k]) * to_f32(a[k]);
    acc = wave_sum(acc);
    if (lane == 0) h[j] = acc * p.scaling;
  }
  __syncthreads();
  const T* B = static_cast<const T*>(sl.b) + static_cast<int64_t>(s) * sl.n * p.r;
  T* y = static_cast<T*>(p.y) + static_cast<int64_t>(t) * p.ys + sl.y_col;
  for (int n = n0 + tid; n < n1; n += kTokThreads) {
    const T* b = B + static_cast<int64_t>(n) * p.r;
    float acc = 0.f;
    for (int j = 0; j < eff; ++j) acc += h[j] * to_f32(b[j]);
    y[n] = from_f32<T>(to_f32(y[n]) + acc);
  }
}

struct TokenShrinkParams {
  const void* x; void* out;
  int64_t xs;
  const int32_t* tts;
  int T, K, r, num_slots;
  float scaling;
  const void* a[MLORA_MAX_SLICES];
};

// out[slice, t, :] = scaling * x[t] . A[s]^T, zero for rows without a slot; grid (token, slice)
template <typename T, typename O>
__global__ __launch_bounds__(kTokThreads) void token_shrink_kernel(TokenShrinkParams p) {
  const int t = blockIdx.x, i = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  O* out = static_cast<O*>(p.out) + (static_cast<int64_t>(i) * p.T + t) * p.r;
  const int s = p.tts[t];
  if (s < 0 || s >= p.num_slots) {
    for (int j = tid; j < p.r; j += kTokThreads) out[j] = from_f32<O>(0.f);
    return;
  }
  const T* x = static_cast<const T*>(p.x) + static_cast<int64_t>(t) * p.xs;
  const T* A = static_cast<const T*>(p.a[i]) + static_cast<int64_t>(s) * p.r * p.K;
  for (int j = wave; j < p.r; j += kTokWaves) {
    const T* a = A + static_cast<int64_t>(j) * p.K;
    float acc = 0.f;
    for (int k = lane; k < p.K; k += kWave) acc += to_f32(x[k]) * to_f32(a[k]);
    acc = wave_sum(acc);
    if (lane == 0) out[j] = from_f32<O>(acc * p.scaling);
  }
}

// The same shrink with 128-bit loads and packed dot products: a wavefront per rank row, each
// lane eight consecutive elements of K at a time, then a 64-lane sum.  For 16-bit elements, K a
// multiple of eight and 16-byte aligned rows (what the reference's tiled kernel,
// lora_ops/triton_ops/lora_shrink_op.py:16-101, covers with its BLOCK_K loads).
template <typename T, typename O>
__global__ __launch_bounds__(kTokThreads) void token_shrink_vec_kernel(TokenShrinkParams p) {
  const int t = blockIdx.x, i = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  O* out = static_cast<O*>(p.out) + (static_cast<int64_t>(i) * p.T + t) * p.r;
  const int s = p.tts[t];
  if (s < 0 || s >= p.num_slots) {
    for (int j = tid; j < p.r; j += kTokThreads) out[j] = from_f32<O>(0.f);
    return;
  }
  const T* x = static_cast<const T*>(p.x) + static_cast<int64_t>(t) * p.xs;
  const T* A = static_cast<const T*>(p.a[i]) + static_cast<int64_t>(s) * p.r * p.K;
  const int chunks = p.K / 8;
  for (int j = wave; j < p.r; j += kTokWaves) {
    const T* a = A + static_cast<int64_t>(j) * p.K;
    float acc = 0.f;
    for (int c = lane; c < chunks; c += kWave) {
      Pack8 xv, av;
      xv.raw = load128(x + c * 8);
      av.raw = load128(a + c * 8);
      acc = dot8<T>(xv, av, acc);
    }
    acc = wave_sum(acc);
    if (lane == 0) out[j] = from_f32<O>(acc * p.scaling);
  }
}

struct TokenExpandParams {
  const void* h; void* y;
  int64_t ys;
  const int32_t* tts;
  int T, r, num_slots, nsplit, add_inputs;
  const void* b[MLORA_MAX_SLICES];
  int n[MLORA_MAX_SLICES];
  int col[MLORA_MAX_SLICES];
};

// y[t, col_i + n] (+)= round_T(h[i, t] . B_i[s]^T); grid (token, column split, slice)
template <typename T, typename H>
__global__ __launch_bounds__(kTokThreads) void token_expand_kernel(TokenExpandParams p) {
  __shared__ float h[MLORA_MAX_RANK];
  const int t = blockIdx.x, i = blockIdx.z;
  const int s = p.tts[t];
  if (s < 0 || s >= p.num_slots) return;
  const int N = p.n[i];
  const int chunk = (N + p.nsplit - 1) / p.nsplit;
  const int n0 = blockIdx.y * chunk;
  const int n1 = n0 + chunk < N ? n0 + chunk : N;
  if (n0 >= n1) return;
  const int tid = threadIdx.x;
  const H* hin = static_cast<const H*>(p.h) + (static_cast<int64_t>(i) * p.T + t) * p.r;
  // The intermediate is taken at the weight's precision, as the reference's kernel casts it.
  for (int j = tid; j < p.r; j += kTokThreads) h[j] = to_f32(from_f32<T>(to_f32(hin[j])));
  __syncthreads();
  const T* B = static_cast<const T*>(p.b[i]) + static_cast<int64_t>(s) * N * p.r;
  T* y = static_cast<T*>(p.y) + static_cast<int64_t>(t) * p.ys + p.col[i];
  for (int n = n0 + tid; n < n1; n += kTokThreads) {
    const T* b = B + static_cast<int64_t>(n) * p.r;
    float acc = 0.f;
    for (int j = 0; j < p.r; ++j) acc += h[j] * to_f32(b[j]);
    const T v = from_f32<T>(acc);
    y[n] = p.add_inputs ? from_f32<T>(to_f32(y[n]) + to_f32(v)) : v;
  }
}

// The same expand with 128-bit loads of the B rows: a thread per output column reads its row of r
// elements eight at a time (r a multiple of eight, 16-bit elements, 16-byte aligned rows); the
// roundings are those of the scalar kernel.
template <typename T, typename H>
__global__ __launch_bounds__(kTokThreads) void token_expand_vec_kernel(TokenExpandParams p) {
  __shared__ float h[MLORA_MAX_RANK];
  const int t = blockIdx.x, i = blockIdx.z;
  const int s = p.tts[t];
  if (s < 0 || s >= p.num_slots) return;
  const int N = p.n[i];
  const int chunk = (N + p.nsplit - 1) / p.nsplit;
  const int n0 = blockIdx.y * chunk;
  const int n1 = n0 + chunk < N ? n0 + chunk : N;
  if (n0 >= n1) return;
  const int tid = threadIdx.x;
  const H* hin = static_cast<const H*>(p.h) + (static_cast<int64_t>(i) * p.T + t) * p.r;
  for (int j = tid; j < p.r; j += kTokThreads) h[j] = to_f32(from_f32<T>(to_f32(hin[j])));
  __syncthreads();
  const T* B = static_cast<const T*>(p.b[i]) + static_cast<int64_t>(s) * N * p.r;
  T* y = static_cast<T*>(p.y) + static_cast<int64_t>(t) * p.ys + p.col[i];
  for (int n = n0 + tid; n < n1; n += kTokThreads) {
    const T* b = B + static_cast<int64_t>(n) * p.r;
    float acc = 0.f;
    for (int j = 0; j < p.r; j += 8) {
      Pack8 bv;
      bv.raw = load128(b + j);
      float f[8];
      unpack8<T>(bv, f);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc += h[j + e] * f[e];
    }
    const T v = from_f32<T>(acc);
    y[n] = p.add_inputs ? from_f32<T>(to_f32(y[n]) + to_f32(v)) : v;
  }
}

struct InstallParams {
  void* a_dst; void* b_dst;
  const void* a_src; const void* b_src;
  int64_t a_ss, b_ss;
  int slot, K, N, r, rank;
  float scaling;
};

// One slot of A and B rewritten in a single pass: rows / columns below `rank` are copied
// (B scaled, rounded first to the source type as a tensor-times-scalar product would be),
// the rest are zeroed.
template <typename D, typename S>
__global__ __launch_bounds__(256) void install_kernel(InstallParams p) {
  const int64_t na = static_cast<int64_t>(p.r) * p.K, nb = static_cast<int64_t>(p.N) * p.r;
  D* A = static_cast<D*>(p.a_dst) + static_cast<int64_t>(p.slot) * na;
  D* B = static_cast<D*>(p.b_dst) + static_cast<int64_t>(p.slot) * nb;
  const S* as = static_cast<const S*>(p.a_src);
  const S* bs = static_cast<const S*>(p.b_src);
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < na + nb; i += stride) {
    if (i < na) {
      const int j = static_cast<int>(i / p.K), k = static_cast<int>(i % p.K);
      A[i] = j < p.rank ? from_f32<D>(to_f32(as[j * p.a_ss + k])) : from_f32<D>(0.f);
    } else {
      const int64_t e = i - na;
      const int n = static_cast<int>(e / p.r), j = static_cast<int>(e % p.r);
      B[e] = j < p.rank ? from_f32<D>(to_f32(from_f32<S>(to_f32(bs[n * p.b_ss + j]) * p.scaling))) : from_f32<D>(0.f);
    }
  }
}

int column_splits(int n_max) {
  int s = (n_max + 1023) / 1024;
  return s < 1 ? 1 : (s > 8 ? 8 : s);
}

}  // namespace

int launch_token_add(const MloraAddArgs* a) {
  TokenAddParams p;
  p.x = a->x; p.y = a->y; p.xs = a->x_stride; p.ys = a->y_stride; p.tts = a->token_to_slot;
  p.T = a->num_tokens; p.K = a->k; p.r = a->r; p.num_slots = a->num_slots; p.scaling = a->scaling;
  p.eff_rank = a->effective_rank;
  int n_max = 0;
  for (int i = 0; i < a->num_slices; ++i) { p.slices[i] = a->slices[i]; n_max = a->slices[i].n > n_max ? a->slices[i].n : n_max; }
  p.nsplit = column_splits(n_max);
  dim3 grid(a->num_tokens, p.nsplit, a->num_slices);
  hipStream_t st = static_cast<hipStream_t>(a->stream);
  switch (a->dtype) {
    case MLORA_DTYPE_F32: hipLaunchKernelGGL(token_add_kernel<float>, grid, dim3(kTokThreads), 0, st, p); break;
    case MLORA_DTYPE_F16: hipLaunchKernelGGL(token_add_kernel<_Float16>, grid, dim3(kTokThreads), 0, st, p); break;
    default: hipLaunchKernelGGL(token_add_kernel<__bf16>, grid, dim3(kTokThreads), 0, st, p); break;
  }
  return check_launch("mlora_add_lora(token)");
}

}  // namespace mlora

using namespace mlora;

namespace {

bool valid_dtype(int d) { return d == MLORA_DTYPE_F32 || d == MLORA_DTYPE_F16 || d == MLORA_DTYPE_BF16; }

template <typename T>
void launch_shrink_out(const TokenShrinkParams& p, dim3 grid, int out_dtype, hipStream_t st) {
  switch (out_dtype) {
    case MLORA_DTYPE_F32: hipLaunchKernelGGL((token_shrink_kernel<T, float>), grid, dim3(kTokThreads), 0, st, p); break;
    case MLORA_DTYPE_F16: hipLaunchKernelGGL((token_shrink_kernel<T, _Float16>), grid, dim3(kTokThreads), 0, st, p); break;
    default: hipLaunchKernelGGL((token_shrink_kernel<T, __bf16>), grid, dim3(kTokThreads), 0, st, p); break;
  }
}

template <typename T>
void launch_shrink_vec_out(const TokenShrinkParams& p, dim3 grid, int out_dtype, hipStream_t st) {
  switch (out_dtype) {
    case MLORA_DTYPE_F32: hipLaunchKernelGGL((token_shrink_vec_kernel<T, float>), grid, dim3(kTokThreads), 0, st, p); break;
    case MLORA_DTYPE_F16: hipLaunchKernelGGL((token_shrink_vec_kernel<T, _Float16>), grid, dim3(kTokThreads), 0, st, p); break;
    default: hipLaunchKernelGGL((token_shrink_vec_kernel<T, __bf16>), grid, dim3(kTokThreads), 0, st, p); break;
  }
}

template <typename T>
void launch_expand_vec_h(const TokenExpandParams& p, dim3 grid, int h_dtype, hipStream_t st) {
  switch (h_dtype) {
    case MLORA_DTYPE_F32: hipLaunchKernelGGL((token_expand_vec_kernel<T, float>), grid, dim3(kTokThreads), 0, st, p); break;
    case MLORA_DTYPE_F16: hipLaunchKernelGGL((token_expand_vec_kernel<T, _Float16>), grid, dim3(kTokThreads), 0, st, p); break;
    default: hipLaunchKernelGGL((token_expand_vec_kernel<T, __bf16>), grid, dim3(kTokThreads), 0, st, p); break;
  }
}

bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; }

template <typename T>
void launch_expand_h(const TokenExpandParams& p, dim3 grid, int h_dtype, hipStream_t st) {
  switch (h_dtype) {
    case MLORA_DTYPE_F32: hipLaunchKernelGGL((token_expand_kernel<T, float>), grid, dim3(kTokThreads), 0, st, p); break;
    case MLORA_DTYPE_F16: hipLaunchKernelGGL((token_expand_kernel<T, _Float16>), grid, dim3(kTokThreads), 0, st, p); break;
    default: hipLaunchKernelGGL((token_expand_kernel<T, __bf16>), grid, dim3(kTokThreads), 0, st, p); break;
  }
}

template <typename D>
void launch_install_src(const InstallParams& p, dim3 grid, int src_dtype, hipStream_t st) {
  switch (src_dtype) {
    case MLORA_DTYPE_F32: hipLaunchKernelGGL((install_kernel<D, float>), grid, dim3(256), 0, st, p); break;
    case MLORA_DTYPE_F16: hipLaunchKernelGGL((install_kernel<D, _Float16>), grid, dim3(256), 0, st, p); break;
    default: hipLaunchKernelGGL((install_kernel<D, __bf16>), grid, dim3(256), 0, st, p); break;
  }
}

}  // namespace

extern "C" int mlora_shrink(const MloraShrinkArgs* a) {
  if (!a) { set_error("mlora_shrink: NULL args"); return MLORA_E_INVALID; }
  if (a->num_tokens < 0 || a->k < 0 || a->r < 0 || a->num_slots < 0 || a->num_slices < 0) {
    set_error("mlora_shrink: negative size"); return MLORA_E_INVALID;
  }
  if (!valid_dtype(a->dtype) || !valid_dtype(a->out_dtype)) { set_error("mlora_shrink: unknown dtype"); return MLORA_E_INVALID; }
  if (a->num_slices > MLORA_MAX_SLICES) { set_error("mlora_shrink: %d slices exceed %d", a->num_slices, MLORA_MAX_SLICES); return MLORA_E_TOO_LARGE; }
  if (a->num_tokens == 0 || a->num_slices == 0 || a->r == 0) return 0;
  if (!a->x || !a->out || !a->token_to_slot) { set_error("mlora_shrink: NULL tensor pointer"); return MLORA_E_INVALID; }
  TokenShrinkParams p;
  p.x = a->x; p.out = a->out; p.xs = a->x_stride; p.tts = a->token_to_slot;
  p.T = a->num_tokens; p.K = a->k; p.r = a->r; p.num_slots = a->num_slots; p.scaling = a->scaling;
  for (int i = 0; i < a->num_slices; ++i) {
    if (!a->a[i]) { set_error("mlora_shrink: NULL A pointer for slice %d", i); return MLORA_E_INVALID; }
    p.a[i] = a->a[i];
  }
  dim3 grid(a->num_tokens, a->num_slices);
  hipStream_t st = static_cast<hipStream_t>(a->stream);
  bool vec = a->dtype != MLORA_DTYPE_F32 && a->k % 8 == 0 && a->x_stride % 8 == 0 && aligned16(a->x);
  for (int i = 0; i < a->num_slices; ++i) vec = vec && aligned16(a->a[i]);
  switch (a->dtype) {
    case MLORA_DTYPE_F32: launch_shrink_out<float>(p, grid, a->out_dtype, st); break;
    case MLORA_DTYPE_F16: vec ? launch_shrink_vec_out<_Float16>(p, grid, a->out_dtype, st) : launch_shrink_out<_Float16>(p, grid, a->out_dtype, st); break;
    default: vec ? launch_shrink_vec_out<__bf16>(p, grid, a->out_dtype, st) : launch_shrink_out<__bf16>(p, grid, a->out_dtype, st); break;
  }
  return check_launch("mlora_shrink");
}

extern "C" int mlora_expand(const MloraExpandArgs* a) {
  if (!a) { set_error("mlora_expand: NULL args"); return MLORA_E_INVALID; }
  if (a->num_tokens < 0 || a->r < 0 || a->num_slots < 0 || a->num_slices < 0 || a->offset_start < 0) {
    set_error("mlora_expand: negative size"); return MLORA_E_INVALID;
  }
  if (!valid_dtype(a->dtype) || !valid_dtype(a->h_dtype)) { set_error("mlora_expand: unknown dtype"); return MLORA_E_INVALID; }
  if (a->num_slices > MLORA_MAX_SLICES) { set_error("mlora_expand: %d slices exceed %d", a->num_slices, MLORA_MAX_SLICES); return MLORA_E_TOO_LARGE; }
  if (a->r > MLORA_MAX_RANK) { set_error("mlora_expand: rank %d exceeds %d", a->r, MLORA_MAX_RANK); return MLORA_E_TOO_LARGE; }
  if (a->num_tokens == 0 || a->num_slices == 0) return 0;
  if (!a->h || !a->y || !a->token_to_slot) { set_error("mlora_expand: NULL tensor pointer"); return MLORA_E_INVALID; }
  TokenExpandParams p;
  p.h = a->h; p.y = a->y; p.ys = a->y_stride; p.tts = a->token_to_slot;
  p.T = a->num_tokens; p.r = a->r; p.num_slots = a->num_slots; p.add_inputs = a->add_inputs ? 1 : 0;
  int col = a->offset_start, n_max = 0;
  for (int i = 0; i < a->num_slices; ++i) {
    if (!a->b[i] || a->n[i] < 0) { set_error("mlora_expand: bad B slice %d", i); return MLORA_E_INVALID; }
    p.b[i] = a->b[i]; p.n[i] = a->n[i]; p.col[i] = col; col += a->n[i];
    n_max = a->n[i] > n_max ? a->n[i] : n_max;
  }
  if (n_max == 0) return 0;
  p.nsplit = column_splits(n_max);
  dim3 grid(a->num_tokens, p.nsplit, a->num_slices);
  hipStream_t st = static_cast<hipStream_t>(a->stream);
  bool vec = a->dtype != MLORA_DTYPE_F32 && a->r % 8 == 0;
  for (int i = 0; i < a->num_slices; ++i) vec = vec && aligned16(a->b[i]);
  switch (a->dtype) {
    case MLORA_DTYPE_F32: launch_expand_h<float>(p, grid, a->h_dtype, st); break;
    case MLORA_DTYPE_F16: vec ? launch_expand_vec_h<_Float16>(p, grid, a->h_dtype, st) : launch_expand_h<_Float16>(p, grid, a->h_dtype, st); break;
    default: vec ? launch_expand_vec_h<__bf16>(p, grid, a->h_dtype, st) : launch_expand_h<__bf16>(p, grid, a->h_dtype, st); break;
  }
  return check_launch("mlora_expand");
}

extern "C" int mlora_install_slot(const MloraInstallArgs* a) {
  if (!a) { set_error("mlora_install_slot: NULL args"); return MLORA_E_INVALID; }
  if (a->slot < 0 || a->k < 0 || a->n < 0 || a->r < 0 || a->rank < 0 || a->rank > a->r) {
    set_error("mlora_install_slot: bad sizes (slot=%d k=%d n=%d r=%d rank=%d)", a->slot, a->k, a->n, a->r, a->rank);
    return MLORA_E_INVALID;
  }
  if (a->slot >= a->num_slots) {
    set_error("mlora_install_slot: slot %d is outside the %d slots of the buffers", a->slot, a->num_slots);
    return MLORA_E_INVALID;
  }
  if (a->rank > 0 && (a->a_src_stride < a->k || a->b_src_stride < a->rank)) {
    set_error("mlora_install_slot: source row strides (%lld, %lld) are shorter than the rows they carry (%d, %d)",
              static_cast<long long>(a->a_src_stride), static_cast<long long>(a->b_src_stride), a->k, a->rank);
    return MLORA_E_INVALID;
  }
  if (!valid_dtype(a->dtype) || !valid_dtype(a->src_dtype)) { set_error("mlora_install_slot: unknown dtype"); return MLORA_E_INVALID; }
  if (!a->a_dst || !a->b_dst || (a->rank > 0 && (!a->a_src || !a->b_src))) { set_error("mlora_install_slot: NULL pointer"); return MLORA_E_INVALID; }
  const int64_t total = static_cast<int64_t>(a->r) * a->k + static_cast<int64_t>(a->n) * a->r;
  if (total == 0) return 0;
  InstallParams p;
  p.a_dst = a->a_dst; p.b_dst = a->b_dst; p.a_src = a->a_src; p.b_src = a->b_src;
  p.a_ss = a->a_src_stride; p.b_ss = a->b_src_stride;
  p.slot = a->slot; p.K = a->k; p.N = a->n; p.r = a->r; p.rank = a->rank; p.scaling = a->scaling;
  int64_t blocks = (total + 255) / 256;
  if (blocks > 2048) blocks = 2048;
  dim3 grid(static_cast<unsigned>(blocks));
  hipStream_t st = static_cast<hipStream_t>(a->stream);
  switch (a->dtype) {
    case MLORA_DTYPE_F32: launch_install_src<float>(p, grid, a->src_dtype, st); break;
    case MLORA_DTYPE_F16: launch_install_src<_Float16>(p, grid, a->src_dtype, st); break;
    default: launch_install_src<__bf16>(p, grid, a->src_dtype, st); break;
  }
  return check_launch("mlora_install_slot");
}
