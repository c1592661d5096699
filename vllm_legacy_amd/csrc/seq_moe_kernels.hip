// Mixture-of-experts feed-forward in the activation dtype (no quantization), routed on the device
// without a host synchronisation:
//   moe_route      per token: router logits in fp32 (plus a bias), softmax over all experts, choice by score plus
//                  a per-expert correction, weights = chosen scores renormalized; also the sigmoid
//                  gate of a shared expert
//   moe_plan       groups the (token, choice) pairs by expert into row tiles of kTile rows (groups
//                  are padded to whole tiles, so a tile belongs to one expert)
//   grouped_linear out[row] = act(W_e a[row]) for the rows of every tile, W_e the tile's expert;
//                  the rows of the first product are gathered from the tokens on the fly
//   moe_combine    per token: weighted sum of its experts' rows (a choice without a row is an
//                  identity expert: the token's own input), plus the gated shared expert
// A row's result does not depend on which other rows share its tile or on where the plan put it.
#include <atomic>

#include "seq_common.h"

namespace vla {
namespace seq {
namespace {

constexpr int kTile = 32;
std::atomic<int> g_grouped_form{0};
constexpr int kMaxRouted = 512;   // experts a router chooses among, identity experts included

__device__ __forceinline__ float act_apply(float z, int act) {
  switch (act) {
    case VLA_ACT_NONE: return z;
    case VLA_ACT_RELU: return fmaxf(z, 0.f);
    case VLA_ACT_RELU2: {
      const float r = fmaxf(z, 0.f);
      return r * r;
    }
    case VLA_ACT_SILU: return z / (1.f + expf(-z));
    default: return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
  }
}

// One workgroup per token.  The logits come from the caller (a matrix product over many tokens) or
// are formed here, a router row per wave at a time.
template <class S>
__global__ __launch_bounds__(256) void moe_route_kernel(
    const typename S::T* __restrict__ h, int64_t h_stride, const float* __restrict__ router,
    const float* __restrict__ logits, int64_t logits_stride, const float* __restrict__ bias,
    const float* __restrict__ correction,
    const float* __restrict__ shared_gate_w, int* __restrict__ experts, float* __restrict__ weights,
    float* __restrict__ shared_gate, int width, int routed, int top) {
  __shared__ float z[kMaxRouted + 1];
  const int t = blockIdx.x, lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const bool gated = shared_gate != nullptr;
  const int rows = routed + (gated ? 1 : 0);
  if (logits != nullptr) {
    for (int n = threadIdx.x; n < rows; n += 256)
      z[n] = logits[(int64_t)t * logits_stride + n] + (bias != nullptr && n < routed ? bias[n] : 0.f);
  } else {
    const typename S::T* hr = h + (int64_t)t * h_stride;
    for (int n = w; n < rows; n += 4) {
      const float* wr = n < routed ? router + (int64_t)n * width : shared_gate_w;
      float dot = 0.f;
      for (int c = lane; c < width; c += kWave) dot += wr[c] * S::to_f32(hr[c]);
      dot = wave_sum(dot);
      if (lane == 0) z[n] = dot + (bias != nullptr && n < routed ? bias[n] : 0.f);
    }
  }
  __syncthreads();
  if (w != 0) return;
  if (gated && lane == 0) shared_gate[t] = 1.f / (1.f + expf(-z[routed]));
  constexpr int PER = kMaxRouted / kWave;
  float s[PER], choice[PER];
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int n = lane + i * kWave;
    s[i] = n < routed ? z[n] : -INFINITY;
    mx = fmaxf(mx, s[i]);
  }
  mx = wave_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    s[i] = lane + i * kWave < routed ? expf(s[i] - mx) : 0.f;
    sum += s[i];
  }
  sum = wave_sum(sum);
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int n = lane + i * kWave;
    s[i] /= sum;
    choice[i] = n < routed ? s[i] + (correction != nullptr ? correction[n] : 0.f) : -INFINITY;
  }
  float total = 0.f, mine = 0.f;     // lane k keeps the k-th chosen score
  int mine_e = 0;
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY, best_s = 0.f;
    int best_n = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int n = lane + i * kWave;
      if (choice[i] > best) {      // ascending n within a lane: the lowest index wins a tie
        best = choice[i];
        best_n = n;
        best_s = s[i];
      }
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
      const float ob = __shfl_xor(best, m, 64), os = __shfl_xor(best_s, m, 64);
      const int on = __shfl_xor(best_n, m, 64);
      if (ob > best || (ob == best && on < best_n)) {
        best = ob;
        best_n = on;
        best_s = os;
      }
    }
#pragma unroll
    for (int i = 0; i < PER; ++i)
      if (lane + i * kWave == best_n) choice[i] = -INFINITY;
    total += best_s;
    if (lane == k) {
      mine = best_s;
      mine_e = best_n;
    }
  }
  if (lane < top) {
    experts[(int64_t)t * top + lane] = mine_e;
    weights[(int64_t)t * top + lane] = mine / (total + 1e-20f);
  }
}

// One workgroup.  pair_row[pair] = the row of the pair in the grouped order (-1: its expert has no
// weights); row_token[row] = the pair's token (-1: padding); tile_expert[tile] = expert (-1: unused).
__global__ __launch_bounds__(1024) void moe_plan_kernel(
    const int* __restrict__ experts, int num_pairs, int top, int num_experts,
    int* __restrict__ pair_row, int* __restrict__ row_token, int* __restrict__ tile_expert,
    int max_tiles) {
  extern __shared__ int lds[];
  int* count = lds;                      // [num_experts]
  int* offset = lds + num_experts;       // [num_experts + 1], in rows
  int* cursor = offset + num_experts + 1;
  for (int e = threadIdx.x; e < num_experts; e += blockDim.x) count[e] = cursor[e] = 0;
  for (int i = threadIdx.x; i < max_tiles; i += blockDim.x) tile_expert[i] = -1;
  for (int i = threadIdx.x; i < max_tiles * kTile; i += blockDim.x) row_token[i] = -1;
  __syncthreads();
  for (int i = threadIdx.x; i < num_pairs; i += blockDim.x) {
    const int e = experts[i];
    if (e >= 0 && e < num_experts) atomicAdd(&count[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0;
    for (int e = 0; e < num_experts; ++e) {
      offset[e] = at;
      at += (count[e] + kTile - 1) / kTile * kTile;
    }
    offset[num_experts] = at;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < num_experts; e += blockDim.x)
    for (int tile = offset[e] / kTile; tile < offset[e + 1] / kTile && tile < max_tiles; ++tile)
      tile_expert[tile] = e;
  for (int i = threadIdx.x; i < num_pairs; i += blockDim.x) {
    const int e = experts[i];
    int row = -1;
    if (e >= 0 && e < num_experts) {
      row = offset[e] + atomicAdd(&cursor[e], 1);
      if (row < max_tiles * kTile)
        row_token[row] = i / top;
      else
        row = -1;
    }
    pair_row[i] = row;
  }
}

template <class S>
struct Mma;
template <>
struct Mma<BF16> {
  typedef short V4 __attribute__((ext_vector_type(4)));
  static __device__ __forceinline__ f32x16 run(u32x2 a, u32x2 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(__builtin_bit_cast(V4, a), __builtin_bit_cast(V4, b), c,
                                                    0, 0, 0);
  }
};
template <>
struct Mma<F16> {
  typedef _Float16 V4 __attribute__((ext_vector_type(4)));
  static __device__ __forceinline__ f32x16 run(u32x2 a, u32x2 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x8f16(__builtin_bit_cast(V4, a), __builtin_bit_cast(V4, b), c, 0,
                                                0, 0);
  }
};

// 16-bit operands on the matrix cores.  One workgroup per (row tile, 128 output columns); wave w
// takes 32 of the columns.  Both operands are K-contiguous, so a lane's fragment of either is one
// 8-byte load: the weight row n = n0 + c and the activation row c, elements 8 ks + 4 hf .. + 3.
// The product runs transposed (weights as the A operand), so lane (hf, c) ends with row c's
// outputs for columns n0 + (i & 3) + 8 (i >> 2) + 4 hf.
template <class S, class SO>
__global__ __launch_bounds__(256) void grouped_linear_mfma_kernel(
    typename SO::T* __restrict__ out, int64_t out_stride, const typename S::T* __restrict__ a,
    int64_t a_stride, const int* __restrict__ row_token, const typename S::T* __restrict__ weight,
    const int* __restrict__ tile_expert, int n_out, int k_in, int act) {
  using T = typename S::T;
  const int tile = blockIdx.x;
  const int e = tile_expert[tile];
  if (e < 0) return;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int hf = lane >> 5, c = lane & 31;
  const int n0 = blockIdx.y * 128 + w * 32;
  if (n0 >= n_out) return;
  const int row = tile * kTile + c;
  const int src = row_token != nullptr ? row_token[row] : row;
  const T* ar = a + (int64_t)(src < 0 ? 0 : src) * a_stride + 4 * hf;
  const T* wr = weight + ((int64_t)e * n_out + min(n0 + c, n_out - 1)) * k_in + 4 * hf;
  f32x16 acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.f;
  for (int k = 0; k < k_in; k += 8) {
    u32x2 av = *reinterpret_cast<const u32x2*>(ar + k);
    if (src < 0) av = u32x2{0u, 0u};
    const u32x2 wv = *reinterpret_cast<const u32x2*>(wr + k);
    acc = Mma<S>::run(wv, av, acc);
  }
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int n = n0 + (i & 3) + 8 * (i >> 2) + 4 * hf;
    if (n < n_out) out[(int64_t)row * out_stride + n] = SO::from_f32(act_apply(acc[i], act));
  }
}

// The same product on 32x32x16 MFMAs (k_in a multiple of 16, 16-byte fragments) with up to kRunTiles
// consecutive row tiles per workgroup: tiles of one expert share the weight fragment a wave has in
// registers, so the weights are read once per run of tiles instead of once per tile.  A workgroup
// walks its tiles in runs of equal expert.
constexpr int kRunTiles = 4;

template <class S>
struct Mma16;
template <>
struct Mma16<BF16> {
  static __device__ __forceinline__ f32x16 run(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b),
                                                   c, 0, 0, 0);
  }
};
template <>
struct Mma16<F16> {
  static __device__ __forceinline__ f32x16 run(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c,
                                                  0, 0, 0);
  }
};

template <class S, class SO, int C>
__device__ __forceinline__ void grouped_run(typename SO::T* __restrict__ out, int64_t out_stride,
                                            const typename S::T* __restrict__ a, int64_t a_stride,
                                            const int* __restrict__ row_token,
                                            const typename S::T* __restrict__ wr, int first_tile, int n0,
                                            int n_out, int k_in, int act, int hf, int c) {
  using T = typename S::T;
  const T* ar[C];
  bool live[C];
  f32x16 acc[C];
#pragma unroll
  for (int r = 0; r < C; ++r) {
    const int row = (first_tile + r) * kTile + c;
    const int src = row_token != nullptr ? row_token[row] : row;
    live[r] = src >= 0;
    ar[r] = a + (int64_t)(src < 0 ? 0 : src) * a_stride + 8 * hf;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[r][i] = 0.f;
  }
#pragma unroll 4
  for (int k = 0; k < k_in; k += 16) {
    const u32x4 wv = *reinterpret_cast<const u32x4*>(wr + k);
#pragma unroll
    for (int r = 0; r < C; ++r) {
      u32x4 av = *reinterpret_cast<const u32x4*>(ar[r] + k);
      if (!live[r]) av = u32x4{0u, 0u, 0u, 0u};
      acc[r] = Mma16<S>::run(wv, av, acc[r]);
    }
  }
#pragma unroll
  for (int r = 0; r < C; ++r) {
    const int row = (first_tile + r) * kTile + c;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int n = n0 + (i & 3) + 8 * (i >> 2) + 4 * hf;
      if (n < n_out) out[(int64_t)row * out_stride + n] = SO::from_f32(act_apply(acc[r][i], act));
    }
  }
}

template <class S, class SO>
__global__ __launch_bounds__(256) void grouped_linear_mfma16_kernel(
    typename SO::T* __restrict__ out, int64_t out_stride, const typename S::T* __restrict__ a,
    int64_t a_stride, const int* __restrict__ row_token, const typename S::T* __restrict__ weight,
    const int* __restrict__ tile_expert, int max_tiles, int n_out, int k_in, int act,
    int tiles_per_group) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int hf = lane >> 5, c = lane & 31;
  const int n0 = (blockIdx.y * (blockDim.x >> 6) + w) * 32;
  if (n0 >= n_out) return;
  const int first = blockIdx.x * tiles_per_group;
  const int last = min(first + tiles_per_group, max_tiles);
  int i = first;
  while (i < last) {
    const int e = tile_expert[i];
    if (e < 0) {
      ++i;
      continue;
    }
    int j = i + 1;
    while (j < last && tile_expert[j] == e) ++j;
    const typename S::T* wr = weight + ((int64_t)e * n_out + min(n0 + c, n_out - 1)) * k_in + 8 * hf;
    switch (j - i) {
      case 1: grouped_run<S, SO, 1>(out, out_stride, a, a_stride, row_token, wr, i, n0, n_out, k_in, act, hf, c); break;
      case 2: grouped_run<S, SO, 2>(out, out_stride, a, a_stride, row_token, wr, i, n0, n_out, k_in, act, hf, c); break;
      case 3: grouped_run<S, SO, 3>(out, out_stride, a, a_stride, row_token, wr, i, n0, n_out, k_in, act, hf, c); break;
      default: grouped_run<S, SO, 4>(out, out_stride, a, a_stride, row_token, wr, i, n0, n_out, k_in, act, hf, c); break;
    }
    i = j;
  }
}

// The form for many tiles and k_in a multiple of 64: the activation rows of a run of tiles (up to
// 128 rows) walk through LDS in chunks of 64 values, staged once for the four waves of the
// workgroup (double-buffered, one barrier per chunk, loaded one chunk ahead); a wave's weight
// fragments still come straight from memory (no other wave wants them), one 16-byte load per 16
// values and 32 columns, used for every tile of the run.
constexpr int kChunk = 64;
constexpr int kARow = kChunk + 8;     // elements: 144-byte rows, 16 lanes' 16-byte reads fall into different banks

template <class S, class SO, int C>
__device__ __forceinline__ void grouped_run_lds(typename S::T* __restrict__ a_lds,
                                                typename SO::T* __restrict__ out, int64_t out_stride,
                                                const typename S::T* __restrict__ a, int64_t a_stride,
                                                const int* __restrict__ row_token,
                                                const typename S::T* __restrict__ wr, int first_tile, int n0,
                                                int n_out, int k_in, int act, int hf, int c) {
  using T = typename S::T;
  const int tid = threadIdx.x;
  // staging: C pieces of 16 bytes per thread and chunk; piece p = tid + 256 u is row p / 8, values 8 (p % 8) ..
  const T* src[C];
#pragma unroll
  for (int u = 0; u < C; ++u) {
    const int p = tid + 256 * u;
    const int row = first_tile * kTile + p / 8;
    const int tok = row_token != nullptr ? row_token[row] : row;
    src[u] = tok < 0 ? nullptr : a + (int64_t)tok * a_stride + 8 * (p % 8);
  }
  u32x4 xa[C];
  auto fetch = [&](int ch) {
#pragma unroll
    for (int u = 0; u < C; ++u)
      xa[u] = src[u] != nullptr ? *reinterpret_cast<const u32x4*>(src[u] + ch * kChunk) : u32x4{0u, 0u, 0u, 0u};
  };
  auto land = [&](int buf) {
#pragma unroll
    for (int u = 0; u < C; ++u) {
      const int p = tid + 256 * u;
      *reinterpret_cast<u32x4*>(a_lds + (size_t)buf * 4 * kTile * kARow + (p / 8) * kARow + 8 * (p % 8)) = xa[u];
    }
  };
  f32x16 acc[C];
#pragma unroll
  for (int r = 0; r < C; ++r)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[r][i] = 0.f;
  const int chunks = k_in / kChunk;
  fetch(0);
  land(0);
  if (chunks > 1) fetch(1);
  __syncthreads();
  for (int ch = 0; ch < chunks; ++ch) {
    const T* tile = a_lds + (size_t)(ch & 1) * 4 * kTile * kARow + c * kARow + 8 * hf;
    u32x4 wv[kChunk / 16];
#pragma unroll
    for (int ks = 0; ks < kChunk / 16; ++ks) wv[ks] = *reinterpret_cast<const u32x4*>(wr + ch * kChunk + 16 * ks);
#pragma unroll
    for (int ks = 0; ks < kChunk / 16; ++ks)
#pragma unroll
      for (int r = 0; r < C; ++r) {
        const u32x4 av = *reinterpret_cast<const u32x4*>(tile + r * kTile * kARow + 16 * ks);
        acc[r] = Mma16<S>::run(wv[ks], av, acc[r]);
      }
    if (ch + 1 < chunks) land((ch + 1) & 1);
    if (ch + 2 < chunks) fetch(ch + 2);
    __syncthreads();
  }
  if (n0 >= n_out) return;
#pragma unroll
  for (int r = 0; r < C; ++r) {
    const int row = (first_tile + r) * kTile + c;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int n = n0 + (i & 3) + 8 * (i >> 2) + 4 * hf;
      if (n < n_out) out[(int64_t)row * out_stride + n] = SO::from_f32(act_apply(acc[r][i], act));
    }
  }
}

template <class S, class SO>
__global__ __launch_bounds__(256) void grouped_linear_lds_kernel(
    typename SO::T* __restrict__ out, int64_t out_stride, const typename S::T* __restrict__ a,
    int64_t a_stride, const int* __restrict__ row_token, const typename S::T* __restrict__ weight,
    const int* __restrict__ tile_expert, int max_tiles, int n_out, int k_in, int act) {
  __shared__ __align__(16) typename S::T a_lds[2 * 4 * kTile * kARow];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int hf = lane >> 5, c = lane & 31;
  const int n0 = blockIdx.y * 128 + w * 32;        // waves past the last column still stage and wait
  const int first = blockIdx.x * kRunTiles;
  const int last = min(first + kRunTiles, max_tiles);
  int i = first;
  while (i < last) {
    const int e = tile_expert[i];
    if (e < 0) {
      ++i;
      continue;
    }
    int j = i + 1;
    while (j < last && tile_expert[j] == e) ++j;
    const typename S::T* wr = weight + ((int64_t)e * n_out + min(n0 + c, n_out - 1)) * k_in + 8 * hf;
    switch (j - i) {
      case 1: grouped_run_lds<S, SO, 1>(a_lds, out, out_stride, a, a_stride, row_token, wr, i, n0, n_out, k_in, act, hf, c); break;
      case 2: grouped_run_lds<S, SO, 2>(a_lds, out, out_stride, a, a_stride, row_token, wr, i, n0, n_out, k_in, act, hf, c); break;
      case 3: grouped_run_lds<S, SO, 3>(a_lds, out, out_stride, a, a_stride, row_token, wr, i, n0, n_out, k_in, act, hf, c); break;
      default: grouped_run_lds<S, SO, 4>(a_lds, out, out_stride, a, a_stride, row_token, wr, i, n0, n_out, k_in, act, hf, c); break;
    }
    i = j;
  }
}

// Any dtype and size, fp32 arithmetic: wave w of a workgroup takes eight rows of the tile, lane =
// output column.
template <class S, class SO>
__global__ __launch_bounds__(256) void grouped_linear_kernel(
    typename SO::T* __restrict__ out, int64_t out_stride, const typename S::T* __restrict__ a,
    int64_t a_stride, const int* __restrict__ row_token, const typename S::T* __restrict__ weight,
    const int* __restrict__ tile_expert, int n_out, int k_in, int act) {
  using T = typename S::T;
  const int tile = blockIdx.x;
  const int e = tile_expert[tile];
  if (e < 0) return;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int n = blockIdx.y * kWave + lane;
  const T* wr = weight + ((int64_t)e * n_out + min(n, n_out - 1)) * k_in;
  const T* ar[8];
  bool live[8];
  float acc[8];
#pragma unroll
  for (int r = 0; r < 8; ++r) {
    const int row = tile * kTile + w * 8 + r;
    const int src = row_token != nullptr ? row_token[row] : row;
    live[r] = src >= 0;
    ar[r] = a + (int64_t)(src < 0 ? 0 : src) * a_stride;
    acc[r] = 0.f;
  }
  for (int k = 0; k < k_in; ++k) {
    const float wv = S::to_f32(wr[k]);
#pragma unroll
    for (int r = 0; r < 8; ++r) acc[r] += wv * S::to_f32(ar[r][k]);
  }
  if (n >= n_out) return;
#pragma unroll
  for (int r = 0; r < 8; ++r) {
    const int row = tile * kTile + w * 8 + r;
    out[(int64_t)row * out_stride + n] = SO::from_f32(act_apply(live[r] ? acc[r] : 0.f, act));
  }
}

template <class S>
__global__ __launch_bounds__(256) void moe_combine_kernel(
    float* __restrict__ out, const float* __restrict__ y, const int* __restrict__ pair_row,
    const float* __restrict__ weights, const typename S::T* __restrict__ h, int64_t h_stride,
    const float* __restrict__ shared_y, const float* __restrict__ shared_gate, int width, int top) {
  const int64_t t = blockIdx.x;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    float acc = 0.f;
    for (int k = 0; k < top; ++k) {
      const int row = pair_row[t * top + k];
      const float v = row >= 0 ? y[(int64_t)row * width + c] : S::to_f32(h[t * h_stride + c]);
      acc += weights[t * top + k] * v;
    }
    if (shared_y != nullptr)
      acc += (shared_gate != nullptr ? shared_gate[t] : 1.f) * shared_y[t * width + c];
    out[t * width + c] = acc;
  }
}

template <class F>
int with_io_dtypes(int a, int b, F&& f) {
  return with_dtype(a, [&](auto sa) { return with_dtype(b, [&](auto sb) { return f(sa, sb); }); });
}

}  // namespace
}  // namespace seq
}  // namespace vla

using namespace vla;
using namespace vla::seq;

extern "C" int vla_seq_moe_route(const void* h, int64_t h_stride, const float* router,
                                 const float* logits, int64_t logits_stride, const float* bias,
                                 const float* correction, const float* shared_gate_weight,
                                 int* experts, float* weights, float* shared_gate, int num_tokens,
                                 int width, int routed, int top, int dtype, void* stream) {
  if (num_tokens == 0) return VLA_OK;
  const bool gated = shared_gate != nullptr;
  if (!experts || !weights || num_tokens < 0 || width <= 0 || routed <= 0 || routed > kMaxRouted ||
      top <= 0 || top > routed || top > kWave ||
      (logits ? logits_stride < routed + (gated ? 1 : 0)
              : (!h || !router || h_stride < width || (gated && !shared_gate_weight))))
    return VLA_ERR_ARG;
  return with_dtype(dtype, [&](auto s) {
    using S = decltype(s);
    moe_route_kernel<S><<<num_tokens, 256, 0, (hipStream_t)stream>>>(
        (const typename S::T*)h, h_stride, router, logits, logits_stride, bias, correction,
        shared_gate_weight, experts, weights, shared_gate, width, routed, top);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}

extern "C" int vla_seq_moe_tile_rows(void) { return kTile; }

extern "C" int vla_seq_moe_plan(const int* experts, int num_tokens, int top, int num_experts,
                                int* pair_row, int* row_token, int* tile_expert, int max_tiles,
                                void* stream) {
  if (!experts || !pair_row || !row_token || !tile_expert || num_tokens < 0 || top <= 0 ||
      num_experts <= 0 || num_experts > 4096 || max_tiles <= 0)
    return VLA_ERR_ARG;
  const size_t lds = sizeof(int) * (3 * (size_t)num_experts + 1);
  moe_plan_kernel<<<1, 1024, lds, (hipStream_t)stream>>>(experts, num_tokens * top, top, num_experts,
                                                        pair_row, row_token, tile_expert, max_tiles);
  VLA_SEQ_HIP_CHECK(hipGetLastError());
  return VLA_OK;
}

extern "C" int vla_seq_grouped_linear(void* out, int64_t out_stride, int out_dtype, const void* a,
                                      int64_t a_stride, const int* row_token, const void* weight,
                                      const int* tile_expert, int max_tiles, int n_out, int k_in,
                                      int act, int dtype, void* stream) {
  if (max_tiles == 0) return VLA_OK;
  if (!out || !a || !weight || !tile_expert || max_tiles < 0 || n_out <= 0 || k_in <= 0 ||
      out_stride < n_out || a_stride < k_in || act < VLA_ACT_NONE || act > VLA_ACT_GELU_TANH)
    return VLA_ERR_ARG;
  return with_io_dtypes(dtype, out_dtype, [&](auto s, auto so) {
    using S = decltype(s);
    using SO = decltype(so);
    using T = typename S::T;
    hipStream_t st = (hipStream_t)stream;
    if constexpr (sizeof(T) == 2) {
      if (k_in % 16 == 0 && ((uintptr_t)a % 16) == 0 && (a_stride % 8) == 0 && ((uintptr_t)weight % 16) == 0) {
        // few tiles (decode steps): the launch is bound by reading each expert's weights once, so
        // every (tile, 32 columns) is a one-wave workgroup of its own; many tiles: four waves
        // and runs of tiles that share the weight fragments
        const int form = g_grouped_form.load(std::memory_order_relaxed);
        const bool few = form == 0 ? (int64_t)max_tiles * ((n_out + 127) / 128) <= 1024 : form == 1;
        if (!few && k_in % kChunk == 0) {
          grouped_linear_lds_kernel<S, SO>
              <<<dim3((max_tiles + kRunTiles - 1) / kRunTiles, (n_out + 127) / 128), 256, 0, st>>>(
                  (typename SO::T*)out, out_stride, (const T*)a, a_stride, row_token, (const T*)weight,
                  tile_expert, max_tiles, n_out, k_in, act);
          VLA_SEQ_HIP_CHECK(hipGetLastError());
          return VLA_OK;
        }
        const int waves = few ? 1 : 4, per = few ? 1 : kRunTiles;
        grouped_linear_mfma16_kernel<S, SO>
            <<<dim3((max_tiles + per - 1) / per, (n_out + 32 * waves - 1) / (32 * waves)), 64 * waves, 0, st>>>(
                (typename SO::T*)out, out_stride, (const T*)a, a_stride, row_token, (const T*)weight,
                tile_expert, max_tiles, n_out, k_in, act, per);
        VLA_SEQ_HIP_CHECK(hipGetLastError());
        return VLA_OK;
      }
      if (k_in % 8 == 0 && ((uintptr_t)a % 8) == 0 && (a_stride % 4) == 0 && ((uintptr_t)weight % 8) == 0) {
        grouped_linear_mfma_kernel<S, SO><<<dim3(max_tiles, (n_out + 127) / 128), 256, 0, st>>>(
            (typename SO::T*)out, out_stride, (const T*)a, a_stride, row_token, (const T*)weight,
            tile_expert, n_out, k_in, act);
        VLA_SEQ_HIP_CHECK(hipGetLastError());
        return VLA_OK;
      }
    }
    grouped_linear_kernel<S, SO><<<dim3(max_tiles, (n_out + kWave - 1) / kWave), 256, 0, st>>>(
        (typename SO::T*)out, out_stride, (const T*)a, a_stride, row_token, (const T*)weight,
        tile_expert, n_out, k_in, act);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}

extern "C" int vla_seq_moe_combine(float* out, const float* y, const int* pair_row,
                                   const float* weights, const void* h, int64_t h_stride,
                                   const float* shared_y, const float* shared_gate, int num_tokens,
                                   int width, int top, int dtype, void* stream) {
  if (num_tokens == 0) return VLA_OK;
  if (!out || !y || !pair_row || !weights || !h || num_tokens < 0 || width <= 0 || top <= 0 ||
      h_stride < width)
    return VLA_ERR_ARG;
  return with_dtype(dtype, [&](auto s) {
    using S = decltype(s);
    moe_combine_kernel<S><<<num_tokens, 256, 0, (hipStream_t)stream>>>(
        out, y, pair_row, weights, (const typename S::T*)h, h_stride, shared_y, shared_gate, width,
        top);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}

// 0: grouped_linear picks its 16-bit form per shape; 1: always one-wave workgroups; 2: always runs of
// tiles (through LDS when k_in allows).  Tests run all.
extern "C" int vla_seq_set_grouped_linear_form(int mode) {
  if (mode < 0 || mode > 2) return VLA_ERR_ARG;
  g_grouped_form.store(mode, std::memory_order_relaxed);
  return VLA_OK;
}
