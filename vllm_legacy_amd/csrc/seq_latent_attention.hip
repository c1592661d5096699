// Causal softmax attention whose keys and values are up-projections of one cached latent per token.
//
// Per token the cache holds one row [latent (rank) | shared rotated key part (rot)] in the model
// dtype: cache [num_blocks, block_size, rank + rot].  Head h's key is [W_uk,h c | k_rot] and its
// value W_uv,h c, so with q_lat,h = W_uk,h^T q_plain,h (the caller's matrix product)
//   score = (q_lat,h . c + q_rot,h . k_rot) * scale,    o_lat,h = sum_j p_j c_j,
// and the head's output is W_uv,h o_lat,h (the caller's product again): every head reads the same
// rows, nothing per head is cached.  latent_rotary_write norms the step's latents, rotates the
// shared key part and the queries' rotated parts (interleaved pairs, frequencies from a table, sine
// and cosine times a magnitude), and writes the cache rows; the attention kernels then read every
// query row's keys from the cache, so prompts, portions of prompts and decode steps are one case.
// Angles, norms, scores, softmax and the weighted sum are fp32.
//
// latent_attention_kernel: one wave per (token, head), any dtype, rank up to 1024.  A tile is 64
// keys: lane j scores key j against the query held in LDS, the wave reduces max / sum (online
// softmax across tiles), then lane d accumulates sum_j p_j c_j[d] with coalesced reads.
#include "seq_common.h"

namespace vla {
namespace seq {
namespace {

constexpr int kMaxRank = 1024;
constexpr int kAccum = kMaxRank / kWave;
constexpr int kHeadsPerGroup = 4;

__device__ __forceinline__ void turn_scaled(float& a, float& b, float angle, float mag) {
  float s, c;
  sincosf(angle, &s, &c);
  s *= mag;
  c *= mag;
  const float a2 = a * c - b * s;
  b = b * c + a * s;
  a = a2;
}

// One workgroup per token.
template <class S>
__global__ __launch_bounds__(256) void latent_rotary_write_kernel(
    typename S::T* __restrict__ q, int64_t q_stride, int q_head_stride, int q_first,
    const typename S::T* __restrict__ kv, int64_t kv_stride, const float* __restrict__ norm_weight,
    float eps, typename S::T* __restrict__ cache, const int64_t* __restrict__ positions,
    const int64_t* __restrict__ slot_mapping, const float* __restrict__ inv_freq, float magnitude,
    int heads, int rank, int rot, int rot_dims, int64_t num_slots) {
  using T = typename S::T;
  __shared__ float red[16];
  const int t = blockIdx.x;
  const float p = (float)positions[t];
  const int half = rot_dims / 2;        // pairs that turn; what follows them passes unchanged
  T* qr = q + (int64_t)t * q_stride + q_first;
  for (int i = threadIdx.x; i < heads * half; i += blockDim.x) {
    const int h = i / half, f = i - h * half;
    T* e = qr + (int64_t)h * q_head_stride + 2 * f;
    float a = S::to_f32(e[0]), b = S::to_f32(e[1]);
    turn_scaled(a, b, p * inv_freq[f], magnitude);
    e[0] = S::from_f32(a);
    e[1] = S::from_f32(b);
  }
  const int64_t slot = slot_mapping[t];
  const bool cached = slot >= 0 && slot < num_slots;    // uniform over the workgroup
  if (!cached) return;
  const T* kr = kv + (int64_t)t * kv_stride;
  T* row = cache + slot * (int64_t)(rank + rot);
  float ss = 0.f;
  for (int c = threadIdx.x; c < rank; c += blockDim.x) {
    const float v = S::to_f32(kr[c]);
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)rank + eps);
  for (int c = threadIdx.x; c < rank; c += blockDim.x)
    row[c] = S::from_f32(S::to_f32(kr[c]) * inv * norm_weight[c]);
  for (int f = threadIdx.x; f < half; f += blockDim.x) {
    float a = S::to_f32(kr[rank + 2 * f]), b = S::to_f32(kr[rank + 2 * f + 1]);
    turn_scaled(a, b, p * inv_freq[f], magnitude);
    row[rank + 2 * f] = S::from_f32(a);
    row[rank + 2 * f + 1] = S::from_f32(b);
  }
  for (int c = 2 * half + threadIdx.x; c < rot; c += blockDim.x) row[rank + c] = kr[rank + c];
}

template <class S>
struct LatentQuery {
  const typename S::T* lat;     // [.., rank]
  int64_t lat_token_stride, lat_head_stride;
  const typename S::T* rot;     // [.., rot]
  int64_t rot_token_stride, rot_head_stride;
};

template <class S>
__global__ __launch_bounds__(kWave* kHeadsPerGroup) void latent_attention_kernel(
    typename S::T* __restrict__ out, int64_t out_token_stride, int64_t out_head_stride,
    LatentQuery<S> q, const typename S::T* __restrict__ cache, const int* __restrict__ block_tables,
    int max_blocks, const int* __restrict__ token_seq, const int64_t* __restrict__ positions,
    int heads, int rank, int rot, int block_size, int num_blocks, float scale) {
  extern __shared__ float lds[];
  const int width = rank + rot;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  float* q_lds = lds + w * width;
  float* p_lds = lds + kHeadsPerGroup * width + w * kWave;
  const int t = blockIdx.x;
  const int h = blockIdx.y * kHeadsPerGroup + w;
  if (h >= heads) return;  // whole wave; no workgroup barrier below
  const int p = (int)positions[t];
  const int* table = block_tables + (int64_t)token_seq[t] * max_blocks;
  for (int d = lane; d < rank; d += kWave)
    q_lds[d] = S::to_f32(q.lat[(int64_t)t * q.lat_token_stride + (int64_t)h * q.lat_head_stride + d]) * scale;
  for (int d = lane; d < rot; d += kWave)
    q_lds[rank + d] =
        S::to_f32(q.rot[(int64_t)t * q.rot_token_stride + (int64_t)h * q.rot_head_stride + d]) * scale;
  wave_sync();
  // a block id outside the pool (a table the host filled wrongly) reads block 0 instead of faulting
  auto token_row = [&](int j) {
    int b = table[j / block_size];
    b = (unsigned)b < (unsigned)num_blocks ? b : 0;
    return cache + ((int64_t)b * block_size + j % block_size) * width;
  };
  float acc[kAccum];
#pragma unroll
  for (int c = 0; c < kAccum; ++c) acc[c] = 0.f;
  float m = -INFINITY, l = 0.f;
  for (int j0 = 0; j0 <= p; j0 += kWave) {
    const int j = j0 + lane;
    float s = -INFINITY;
    if (j <= p) {
      const typename S::T* kr = token_row(j);
      float dot = 0.f;
      for (int d = 0; d < width; ++d) dot += q_lds[d] * S::to_f32(kr[d]);
      s = dot;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float pj = j <= p ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);  // first tile: exp(-inf) = 0
    l = l * corr + wave_sum(pj);
    m = m_new;
    wave_sync();
    p_lds[lane] = pj;
    wave_sync();
#pragma unroll
    for (int c = 0; c < kAccum; ++c) acc[c] *= corr;
    const int n = min(kWave, p - j0 + 1);
    for (int jj = 0; jj < n; ++jj) {
      const typename S::T* vr = token_row(j0 + jj);
      const float pv = p_lds[jj];
#pragma unroll
      for (int c = 0; c < kAccum; ++c) {
        const int d = lane + c * kWave;
        if (d < rank) acc[c] += pv * S::to_f32(vr[d]);
      }
    }
  }
  const float inv = 1.f / l;
  typename S::T* orow = out + (int64_t)t * out_token_stride + (int64_t)h * out_head_stride;
#pragma unroll
  for (int c = 0; c < kAccum; ++c) {
    const int d = lane + c * kWave;
    if (d < rank) orow[d] = S::from_f32(acc[c] * inv);
  }
}

}  // namespace
}  // namespace seq
}  // namespace vla

using namespace vla;
using namespace vla::seq;

extern "C" int vla_seq_latent_rotary_write(void* q, int64_t q_stride, int q_head_stride, int q_first,
                                           const void* kv, int64_t kv_stride,
                                           const float* norm_weight, float eps, void* cache,
                                           const int64_t* positions, const int64_t* slot_mapping,
                                           const float* inv_freq, float magnitude, int num_tokens,
                                           int heads, int rank, int rot, int rot_dims,
                                           int block_size, int num_blocks, int dtype,
                                           void* stream) {
  if (num_tokens == 0) return VLA_OK;
  if (!q || !kv || !norm_weight || !cache || !positions || !slot_mapping || num_tokens < 0 ||
      heads <= 0 || rank <= 0 || rot < 0 || rot_dims < 0 || rot_dims > rot || (rot_dims & 1) ||
      (rot_dims > 0 && !inv_freq) || q_first < 0 ||
      q_head_stride < rot || q_stride < (int64_t)(heads - 1) * q_head_stride + q_first + rot ||
      kv_stride < rank + rot || block_size <= 0 || num_blocks <= 0)
    return VLA_ERR_ARG;
  return with_dtype(dtype, [&](auto s) {
    using S = decltype(s);
    using T = typename S::T;
    latent_rotary_write_kernel<S><<<num_tokens, 256, 0, (hipStream_t)stream>>>(
        (T*)q, q_stride, q_head_stride, q_first, (const T*)kv, kv_stride, norm_weight, eps, (T*)cache,
        positions, slot_mapping, inv_freq, magnitude, heads, rank, rot, rot_dims,
        (int64_t)num_blocks * block_size);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}

extern "C" int vla_seq_latent_attention(void* out, int64_t out_token_stride, int64_t out_head_stride,
                                        const void* q_lat, int64_t lat_token_stride,
                                        int64_t lat_head_stride, const void* q_rot,
                                        int64_t rot_token_stride, int64_t rot_head_stride,
                                        const void* cache, const int* block_tables, int max_blocks,
                                        const int* token_seq, const int64_t* positions,
                                        int num_tokens, int heads, int rank, int rot, int block_size,
                                        int num_blocks, float scale, int dtype, void* stream) {
  if (num_tokens == 0) return VLA_OK;
  if (!out || !q_lat || (rot > 0 && !q_rot) || !cache || !block_tables || !token_seq || !positions ||
      num_tokens < 0 || heads <= 0 || rot < 0 || block_size <= 0 || num_blocks <= 0 ||
      max_blocks <= 0)
    return VLA_ERR_ARG;
  if (rank <= 0 || rank > kMaxRank || rot > kMaxRank) return VLA_ERR_HEAD_SIZE;
  return with_dtype(dtype, [&](auto s) {
    using S = decltype(s);
    using T = typename S::T;
    const LatentQuery<S> q{(const T*)q_lat, lat_token_stride, lat_head_stride, (const T*)q_rot,
                           rot_token_stride, rot_head_stride};
    const dim3 grid(num_tokens, (heads + kHeadsPerGroup - 1) / kHeadsPerGroup);
    const size_t lds = (size_t)kHeadsPerGroup * (rank + rot + kWave) * sizeof(float);
    latent_attention_kernel<S><<<grid, kWave * kHeadsPerGroup, lds, (hipStream_t)stream>>>(
        (T*)out, out_token_stride, out_head_stride, q, (const T*)cache, block_tables, max_blocks,
        token_seq, positions, heads, rank, rot, block_size, num_blocks, scale);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}
