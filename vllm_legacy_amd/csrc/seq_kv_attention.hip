// Causal softmax attention over paged key and value caches with rotary positions on queries and
// keys, values that are rotated by their own position when they are cached (the head's output is
// turned back by the query's position), an optional sliding window that may keep a sequence's
// first tokens visible, an optional cap on the scores (cap * tanh(score / cap)) and a sigmoid gate of
// one number per head.  rotary_kv_write can also norm the whole query and key rows before it rotates
// them and blend the values with another layer's values of the same tokens.
//
// With a window and `keep_first` kept tokens, query position p sees j <= p with p - j < window or
// j < keep_first.  The kernels walk such a key set through one index u: with lo the window's first
// key and nk = min(keep_first, lo), u < nk is key u and u >= nk is key lo + u - nk.
//
// Caches: keys [num_blocks, block_size, kv_heads, dim] and values [num_blocks, block_size, kv_heads,
// vdim] in the model dtype, token-major rows.  rotary_kv_write rotates the step's queries in place
// and writes the rotated keys and values to their slots; the attention kernels then read every
// query row's keys from the caches, so prompts, portions of prompts and decode steps are one case
// and a position's result cannot depend on how its sequence was cut into steps.  Angles, scores,
// softmax and the weighted sum are fp32.
//
// kv_attention_kernel: one wave per (token, query head), any dtype and head size up to 256.  A
// tile is 64 keys: lane j scores key j against the query held in LDS, the wave reduces max / sum
// (online softmax across tiles), then lane d accumulates sum_j p_j v_j[d] with coalesced reads.
#include <atomic>

#include "seq_common.h"

namespace vla {
namespace seq {
namespace {

constexpr int kMaxDim = 256;
constexpr int kAccum = kMaxDim / kWave;
constexpr int kHeadsPerGroup = 4;

// the pair (a, b) turned by angle: (a cos - b sin, b cos + a sin)
__device__ __forceinline__ void turn(float& a, float& b, float angle) {
  float s, c;
  sincosf(angle, &s, &c);
  const float a2 = a * c - b * s;
  b = b * c + a * s;
  a = a2;
}

// cap * tanh(s / cap): libm's tanh in the fp32 kernel, one exponential and one reciprocal in the
// matrix-core kernels (absolute error of a few 1e-7 times cap)
__device__ __forceinline__ float cap_score(float s, float cap) { return cap * tanhf(s / cap); }
__device__ __forceinline__ float cap_score_fast(float s, float cap, float two_log2e_over_cap) {
  const float e = __builtin_amdgcn_exp2f(s * two_log2e_over_cap);   // e^(2 s / cap); inf and 0 are fine
  return cap - 2.f * cap * __builtin_amdgcn_rcpf(e + 1.f);
}

// element indices of pair i among `span` rotated elements
__device__ __forceinline__ void pair_index(int i, int span, int interleaved, int& ia, int& ib) {
  if (interleaved) {
    ia = 2 * i;
    ib = 2 * i + 1;
  } else {
    ia = i;
    ib = i + span / 2;
  }
}

// One workgroup per token: every head's rotated pairs, then the elements that are not rotated.
template <class S>
__global__ __launch_bounds__(256) void rotary_kv_write_kernel(
    typename S::T* __restrict__ q, int64_t q_stride, const typename S::T* __restrict__ k,
    int64_t k_stride, const typename S::T* __restrict__ v, int64_t v_stride,
    typename S::T* __restrict__ key_cache, typename S::T* __restrict__ value_cache,
    const int64_t* __restrict__ positions, const int64_t* __restrict__ slot_mapping,
    const float* __restrict__ inv_freq, const float* __restrict__ value_inv_freq, int heads,
    int kv_heads, int dim, int vdim, int rot_dims, int interleaved, int64_t num_slots,
    const float* __restrict__ q_norm, const float* __restrict__ k_norm, float norm_eps,
    const typename S::T* __restrict__ v_other, int64_t v_other_stride,
    const float* __restrict__ v_blend) {
  using T = typename S::T;
  __shared__ float red[16];
  const int t = blockIdx.x;
  const float p = (float)positions[t];
  int64_t slot = slot_mapping[t];
  const bool cached = slot >= 0 && slot < num_slots;
  const int half = rot_dims / 2;
  const int rest = dim - rot_dims;
  T* qr = q + (int64_t)t * q_stride;
  const T* kr = k + (int64_t)t * k_stride;
  // RMS norm over the whole row (all heads at once) with a weight per element, before the rotation
  float q_inv = 1.f, k_inv = 1.f;
  if (q_norm != nullptr) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < heads * dim; i += blockDim.x) {
      const float x = S::to_f32(qr[i]);
      ss += x * x;
    }
    q_inv = 1.f / sqrtf(block_sum(ss, red) / (float)(heads * dim) + norm_eps);
  }
  if (k_norm != nullptr) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < kv_heads * dim; i += blockDim.x) {
      const float x = S::to_f32(kr[i]);
      ss += x * x;
    }
    k_inv = 1.f / sqrtf(block_sum(ss, red) / (float)(kv_heads * dim) + norm_eps);
  }
  for (int i = threadIdx.x; i < heads * half; i += blockDim.x) {
    const int h = i / half, f = i - h * half;
    int ia, ib;
    pair_index(f, rot_dims, interleaved, ia, ib);
    float a = S::to_f32(qr[h * dim + ia]), b = S::to_f32(qr[h * dim + ib]);
    if (q_norm != nullptr) {
      a *= q_inv * q_norm[h * dim + ia];
      b *= q_inv * q_norm[h * dim + ib];
    }
    turn(a, b, p * inv_freq[f]);
    qr[h * dim + ia] = S::from_f32(a);
    qr[h * dim + ib] = S::from_f32(b);
  }
  if (q_norm != nullptr) {
    for (int i = threadIdx.x; i < heads * rest; i += blockDim.x) {
      const int h = i / rest, d = rot_dims + (i - h * rest);
      qr[h * dim + d] = S::from_f32(S::to_f32(qr[h * dim + d]) * q_inv * q_norm[h * dim + d]);
    }
  }
  if (!cached) return;
  T* kc = key_cache + slot * (int64_t)kv_heads * dim;
  for (int i = threadIdx.x; i < kv_heads * half; i += blockDim.x) {
    const int h = i / half, f = i - h * half;
    int ia, ib;
    pair_index(f, rot_dims, interleaved, ia, ib);
    float a = S::to_f32(kr[h * dim + ia]), b = S::to_f32(kr[h * dim + ib]);
    if (k_norm != nullptr) {
      a *= k_inv * k_norm[h * dim + ia];
      b *= k_inv * k_norm[h * dim + ib];
    }
    turn(a, b, p * inv_freq[f]);
    kc[h * dim + ia] = S::from_f32(a);
    kc[h * dim + ib] = S::from_f32(b);
  }
  for (int i = threadIdx.x; i < kv_heads * rest; i += blockDim.x) {
    const int h = i / rest, d = rot_dims + (i - h * rest);
    if (k_norm != nullptr)
      kc[h * dim + d] = S::from_f32(S::to_f32(kr[h * dim + d]) * k_inv * k_norm[h * dim + d]);
    else
      kc[h * dim + d] = kr[h * dim + d];
  }
  const T* vr = v + (int64_t)t * v_stride;
  T* vc = value_cache + slot * (int64_t)kv_heads * vdim;
  if (v_other != nullptr) {
    // the cached value is (1 - lambda) v + lambda v_other, v_other another layer's values of this token
    const float lam = v_blend[0];
    const T* vo = v_other + (int64_t)t * v_other_stride;
    for (int i = threadIdx.x; i < kv_heads * vdim; i += blockDim.x)
      vc[i] = S::from_f32((1.f - lam) * S::to_f32(vr[i]) + lam * S::to_f32(vo[i]));
    return;
  }
  if (value_inv_freq == nullptr) {
    for (int i = threadIdx.x; i < kv_heads * vdim; i += blockDim.x) vc[i] = vr[i];
    return;
  }
  const int vhalf = vdim / 2;
  for (int i = threadIdx.x; i < kv_heads * vhalf; i += blockDim.x) {
    const int h = i / vhalf, f = i - h * vhalf;
    int ia, ib;
    pair_index(f, vdim, interleaved, ia, ib);
    float a = S::to_f32(vr[h * vdim + ia]), b = S::to_f32(vr[h * vdim + ib]);
    turn(a, b, p * value_inv_freq[f]);
    vc[h * vdim + ia] = S::from_f32(a);
    vc[h * vdim + ib] = S::from_f32(b);
  }
  if (vdim & 1) {
    for (int h = threadIdx.x; h < kv_heads; h += blockDim.x)
      vc[h * vdim + vdim - 1] = vr[h * vdim + vdim - 1];
  }
}

// The epilogue every attention kernel of this file shares: o_lds holds one head's normalized
// output [vdim] in fp32; turn pair m back by the query's position, gate, write.
template <class S>
__device__ __forceinline__ void write_head_output(typename S::T* __restrict__ orow,
                                                  const float* __restrict__ o_lds, int vdim, float p,
                                                  const float* __restrict__ out_inv_freq,
                                                  int interleaved, float gate, int first, int step) {
  const int vhalf = vdim / 2;
  for (int d = first; d < vdim; d += step) {
    float val = o_lds[d];
    if (out_inv_freq != nullptr && d < 2 * vhalf) {
      int f, other;
      bool is_a;
      if (interleaved) {
        f = d >> 1;
        is_a = (d & 1) == 0;
        other = d ^ 1;
      } else {
        is_a = d < vhalf;
        f = is_a ? d : d - vhalf;
        other = is_a ? d + vhalf : d - vhalf;
      }
      float s, c;
      sincosf(p * out_inv_freq[f], &s, &c);
      // turned by the negative angle: (a cos + b sin, b cos - a sin)
      val = is_a ? val * c + o_lds[other] * s : val * c - o_lds[other] * s;
    }
    orow[d] = S::from_f32(val * gate);
  }
}

template <class S>
__global__ __launch_bounds__(kWave* kHeadsPerGroup) void kv_attention_kernel(
    typename S::T* __restrict__ out, int64_t out_stride, const typename S::T* __restrict__ q,
    int64_t q_stride, const typename S::T* __restrict__ gate, int64_t gate_stride,
    const typename S::T* __restrict__ key_cache, const typename S::T* __restrict__ value_cache,
    const int* __restrict__ block_tables, int max_blocks, const int* __restrict__ token_seq,
    const int64_t* __restrict__ positions, const float* __restrict__ out_inv_freq, int interleaved,
    int heads, int kv_heads, int dim, int vdim, int block_size, int num_blocks, int window,
    float scale, int keep_first, float softcap) {
  __shared__ float q_lds[kHeadsPerGroup][kMaxDim];
  __shared__ float p_lds[kHeadsPerGroup][kWave];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int t = blockIdx.x;
  const int h = blockIdx.y * kHeadsPerGroup + w;
  if (h >= heads) return;  // whole wave; no workgroup barrier below
  const int g = h / (heads / kv_heads);
  const int p = (int)positions[t];
  const int* table = block_tables + (int64_t)token_seq[t] * max_blocks;
  const int lo = window > 0 ? max(0, p - window + 1) : 0;
  const int nk = min(keep_first, lo);         // kept keys ahead of the window
  const int total = nk + p - lo + 1;
  auto key_of = [&](int u) { return u < nk ? u : u - nk + lo; };
  for (int d = lane; d < dim; d += kWave)
    q_lds[w][d] = S::to_f32(q[(int64_t)t * q_stride + (int64_t)h * dim + d]) * scale;
  wave_sync();
  // a block id outside the pool (a table the host filled wrongly) reads block 0 instead of faulting
  auto token_row = [&](int j) {
    int b = table[j / block_size];
    b = (unsigned)b < (unsigned)num_blocks ? b : 0;
    return ((int64_t)b * block_size + j % block_size) * kv_heads + g;
  };

  float acc[kAccum];
#pragma unroll
  for (int c = 0; c < kAccum; ++c) acc[c] = 0.f;
  float m = -INFINITY, l = 0.f;
  for (int u0 = 0; u0 < total; u0 += kWave) {
    const int u = u0 + lane;
    float s = -INFINITY;
    if (u < total) {
      const typename S::T* kr = key_cache + token_row(key_of(u)) * dim;
      float dot = 0.f;
      for (int d = 0; d < dim; ++d) dot += q_lds[w][d] * S::to_f32(kr[d]);
      s = softcap > 0.f ? cap_score(dot, softcap) : dot;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float pj = u < total ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);  // first tile: exp(-inf) = 0
    l = l * corr + wave_sum(pj);
    m = m_new;
    wave_sync();
    p_lds[w][lane] = pj;
    wave_sync();
#pragma unroll
    for (int c = 0; c < kAccum; ++c) acc[c] *= corr;
    const int n = min(kWave, total - u0);
    for (int jj = 0; jj < n; ++jj) {
      const typename S::T* vr = value_cache + token_row(key_of(u0 + jj)) * vdim;
      const float pv = p_lds[w][jj];
#pragma unroll
      for (int c = 0; c < kAccum; ++c) {
        const int d = lane + c * kWave;
        if (d < vdim) acc[c] += pv * S::to_f32(vr[d]);
      }
    }
  }
  wave_sync();
  const float inv = 1.f / l;
#pragma unroll
  for (int c = 0; c < kAccum; ++c) {
    const int d = lane + c * kWave;
    if (d < vdim) q_lds[w][d] = acc[c] * inv;   // the query is done with
  }
  wave_sync();
  float gv = 1.f;
  if (gate != nullptr) gv = 1.f / (1.f + expf(-S::to_f32(gate[(int64_t)t * gate_stride + h])));
  write_head_output<S>(out + (int64_t)t * out_stride + (int64_t)h * vdim, q_lds[w], vdim, (float)p,
                       out_inv_freq, interleaved, gv, lane, kWave);
}


// ---------------------------------------------------------------------------------------------
// Matrix-core kernels for 16-bit models.  Both products run in transposed form on 32x32x8 MFMAs,
// lane = (hf, c) = (lane >> 5, lane & 31):
//   S^T = K q^T   A = K    lane: key c, dims 8 ks + 4 hf .. + 3
//                 B = q^T  lane: query c, the same dims (registers, loaded once)
//                 C        lane: query c, keys (i & 3) + 8 (i >> 2) + 4 hf, i = 0 .. 15
//   O^T = V^T P^T A = V^T  lane: value dim 32 n + c, keys 8 s + 4 hf .. + 3
//                 B = P^T  lane: query c, the same keys = registers 4 s .. 4 s + 3 of C above
//                 C        lane: query c, dims 32 n + (i & 3) + 8 (i >> 2) + 4 hf
// so a lane owns one query's scores, running max / sum and output column, and both elements of
// every rotated output pair (neighbours when interleaved; vdim / 2 = 16 (vdim / 32) apart
// otherwise, which moves n and i >> 2 but neither hf nor c).  Scores leave the first product in
// fp32 and stay there; a weight enters the second product as the sum of two 16-bit numbers (its
// rounding and the rounding of what the rounding lost).
template <class S>
struct Mfma8;
template <>
struct Mfma8<BF16> {
  typedef short V4 __attribute__((ext_vector_type(4)));
  static __device__ __forceinline__ f32x16 run(u32x2 a, u32x2 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(__builtin_bit_cast(V4, a), __builtin_bit_cast(V4, b), c,
                                                    0, 0, 0);
  }
};
template <>
struct Mfma8<F16> {
  typedef _Float16 V4 __attribute__((ext_vector_type(4)));
  static __device__ __forceinline__ f32x16 run(u32x2 a, u32x2 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x8f16(__builtin_bit_cast(V4, a), __builtin_bit_cast(V4, b), c, 0,
                                                0, 0);
  }
};
template <class S>
__device__ __forceinline__ uint32_t bits16(float v) {
  return (uint32_t)__builtin_bit_cast(uint16_t, S::from_f32(v));
}
template <class S>
__device__ __forceinline__ float from_bits16(uint32_t b) {
  return S::to_f32(__builtin_bit_cast(typename S::T, (uint16_t)b));
}

constexpr int kTile = 32;
std::atomic<int> g_kv_kernel{0};

// dim index of register i of output block n for lane half hf
__device__ __forceinline__ constexpr int out_dim(int n, int i, int hf) {
  return 32 * n + (i & 3) + 8 * (i >> 2) + 4 * hf;
}

// Turns the output pairs a lane holds back by the query's position (o[n][i] normalized already).
template <int VB>
__device__ __forceinline__ void turn_back(f32x16 (&o)[VB], int hf, float p,
                                          const float* __restrict__ out_inv_freq, int interleaved) {
  constexpr int VD = 32 * VB;
  if (interleaved) {
#pragma unroll
    for (int n = 0; n < VB; ++n)
#pragma unroll
      for (int i = 0; i < 16; i += 2) {
        float s, c;
        sincosf(p * out_inv_freq[out_dim(n, i, hf) >> 1], &s, &c);
        const float a = o[n][i], b = o[n][i + 1];
        o[n][i] = a * c + b * s;
        o[n][i + 1] = b * c - a * s;
      }
  } else {
    // partner of dim d < VD / 2 is d + 16 VB: block n + VB / 2 (and, for odd VB, i + 8)
#pragma unroll
    for (int n = 0; n < VB; ++n)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int d = 32 * n + (i & 3) + 8 * (i >> 2);      // without 4 hf: same for both halves
        if (d < VD / 2) {
          const int d2 = d + VD / 2;
          const int n2 = d2 / 32, r2 = d2 % 32;
          const int i2 = (r2 & 3) + 4 * (r2 >> 3);
          float s, c;
          sincosf(p * out_inv_freq[d + 4 * hf], &s, &c);
          const float a = o[n][i], b = o[n2][i2];
          o[n][i] = a * c + b * s;
          o[n2][i2] = b * c - a * s;
        }
      }
  }
}

// kv_attention_tile_kernel<S, DB, VB>: runs of rows (prompts, portions), on 32x32x16 MFMAs.  One
// workgroup per (sequence, tile of query rows, KV head, chunk of its query heads).  Its four waves
// are (query head of the chunk) x (block of 32 consecutive rows): 4 x 1 for groups of three heads
// and more, 2 x 2 for two, 1 x 4 for one, so a tile is 32, 64 or 128 rows.  Keys and values from
// the first row's window start to the last row walk through LDS in tiles of 64, row-major, staged
// once for all waves and loaded one tile ahead; the rows' places in the paged caches are looked up
// once per tile by 64 threads, two tiles ahead.
//   S^T = K q^T   A = K    lane: key c of a 32-key block, dims 16 ks + 8 hf .. + 7   (LDS, 16 bytes)
//                 B = q^T  lane: query c, the same dims (registers, loaded once)
//                 C        lane: query c, keys (i & 3) + 8 (i >> 2) + 4 hf, i = 0 .. 15
//   O^T = V^T P^T B = P^T  lane: query c, registers 8 s .. 8 s + 7 of C = keys 16 s + 4 hf + {0..3, 8..11}
//                 A = V^T  lane: value dim 32 n + c of the same eight keys (two transposing reads
//                          of the row-major tile)
// The k index of the second product is a free relabelling of the keys, so the weights go from the
// first product's result to the second's operand without leaving the lane.  Scores, running
// max / sum (base 2) and the accumulators are fp32; a weight enters the second product rounded to
// the model dtype.
template <class S>
struct Mfma16;
template <>
struct Mfma16<BF16> {
  static __device__ __forceinline__ f32x16 run(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b),
                                                   c, 0, 0, 0);
  }
};
template <>
struct Mfma16<F16> {
  static __device__ __forceinline__ f32x16 run(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c,
                                                  0, 0, 0);
  }
};

constexpr int kKeys = 64;     // keys per staged tile
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef s16x4 __attribute__((address_space(3))) * lds_s16x4;

// two fp32 -> one word of two model-dtype values (round to nearest even), as one packed convert
template <class S>
__device__ __forceinline__ uint32_t pack2(float a, float b);
template <>
__device__ __forceinline__ uint32_t pack2<F16>(float a, float b) {
  const f32x2 v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
}
template <>
__device__ __forceinline__ uint32_t pack2<BF16>(float a, float b) {
  const f32x2 v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}

template <class S, int DB, int VB>
__global__ __launch_bounds__(256, 2) void kv_attention_tile_kernel(
    typename S::T* __restrict__ out, int64_t out_stride, const typename S::T* __restrict__ q,
    int64_t q_stride, const typename S::T* __restrict__ gate, int64_t gate_stride,
    const typename S::T* __restrict__ key_cache, const typename S::T* __restrict__ value_cache,
    const int* __restrict__ block_tables, int max_blocks, const int* __restrict__ query_start_loc,
    const int* __restrict__ context_lens, const float* __restrict__ out_inv_freq, int interleaved,
    int heads, int kv_heads, int block_size, int num_blocks, int window, float scale, int head_waves,
    int keep_first, float softcap) {
  using T = typename S::T;
  using M = Mfma16<S>;
  constexpr int D = 32 * DB, VD = 32 * VB;
  // elements; rows stay 16-byte aligned, and four value rows a transposing read takes fall into
  // different banks
  constexpr int KROW = D + 8, VROW = VD + 16;
  __shared__ __align__(16) T k_lds2[2][kKeys * KROW];  // two tiles: one is read while the next lands
  __shared__ __align__(16) T v_lds2[2][kKeys * VROW];
  __shared__ long long rows_lds[2][kKeys];            // token row of each key of a tile, -1: none
  const int b = blockIdx.z;
  const int row_blocks = 4 / head_waves;              // blocks of 32 query rows per workgroup
  const int tile_rows = kTile * row_blocks;
  // the last tiles of a run have the most keys to walk: they are dispatched first
  const int tile_x = gridDim.x - 1 - blockIdx.x;
  const int t_first = query_start_loc[b] + tile_rows * tile_x;
  const int n_tile = min(tile_rows, query_start_loc[b + 1] - t_first);
  if (n_tile <= 0) return;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int hf = lane >> 5, c = lane & 31;
  const int group = heads / kv_heads;
  const int chunks = (group + head_waves - 1) / head_waves;
  const int g = blockIdx.y / chunks;
  const int h = g * group + (blockIdx.y % chunks) * head_waves + w % head_waves;
  const int rb = w / head_waves;                      // this wave's block of rows
  const int t0 = t_first + kTile * rb;
  const int nq = min(kTile, n_tile - kTile * rb);     // <= 0: no rows for this wave
  const bool active = h < g * group + group && nq > 0;
  const int p_first = context_lens[b] + tile_rows * tile_x, p_last = p_first + n_tile - 1;
  const int p0 = p_first + kTile * rb;                // this wave's first position
  const int pq = p0 + c;
  const int j_lo = window > 0 ? max(0, p_first - window + 1) : 0;
  // the keys this workgroup walks, through one index: the kept first tokens that lie ahead of the
  // first row's window, then the window's first key to the last row
  const int nk = min(keep_first, j_lo);
  const int total = nk + p_last - j_lo + 1;
  auto key_of = [&](int u) { return u < nk ? u : u - nk + j_lo; };
  const int* table = block_tables + (int64_t)b * max_blocks;
  const float scale2 = scale * 1.4426950408889634f;   // scores in base 2
  const float cap2 = softcap * 1.4426950408889634f, cap_arg = softcap > 0.f ? 2.f * 1.4426950408889634f / softcap : 0.f;

  u32x4 qf[D / 16];
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks) {
    u32x4 v = {0u, 0u, 0u, 0u};
    if (active && c < nq)
      v = *reinterpret_cast<const u32x4*>(q + (int64_t)(t0 + c) * q_stride + (int64_t)h * D + 16 * ks + 8 * hf);
    qf[ks] = v;
  }
  f32x16 o[VB];
#pragma unroll
  for (int n = 0; n < VB; ++n)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[n][i] = 0.f;
  float m = -INFINITY, l = 0.f;

  // threads 0 .. 63 look the rows of a tile up: the block id is read one step before it is used
  auto load_block = [&](int u0) {
    const int u = u0 + tid;
    int blk = -1;
    if (u < total) {
      blk = table[key_of(u) / block_size];
      blk = (unsigned)blk < (unsigned)num_blocks ? blk : 0;
    }
    return blk;
  };
  auto store_row = [&](int u0, int blk, int buf) {
    const int j = key_of(u0 + tid);
    rows_lds[buf][tid] = blk < 0 ? -1 : ((long long)blk * block_size + j % block_size) * kv_heads + g;
  };
  // staging: DB + VB pieces of 16 bytes per thread and tile
  u32x4 xk[DB], xv[VB];
  auto fetch = [&](int buf) {
#pragma unroll
    for (int u = 0; u < DB; ++u) {
      const int i = tid + 256 * u;
      const int r = i / (D / 8), v = i % (D / 8);
      const long long row = rows_lds[buf][r];
      const u32x4 got = *reinterpret_cast<const u32x4*>(key_cache + (row >= 0 ? row * D + 8 * v : 0));
      xk[u] = row >= 0 ? got : u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int u = 0; u < VB; ++u) {
      const int i = tid + 256 * u;
      const int r = i / (VD / 8), v = i % (VD / 8);
      const long long row = rows_lds[buf][r];
      const u32x4 got = *reinterpret_cast<const u32x4*>(value_cache + (row >= 0 ? row * VD + 8 * v : 0));
      xv[u] = row >= 0 ? got : u32x4{0u, 0u, 0u, 0u};
    }
  };
  auto land = [&](int buf) {                           // the fetched tile into LDS
#pragma unroll
    for (int u = 0; u < DB; ++u) {
      const int i = tid + 256 * u;
      const int r = i / (D / 8), v = i % (D / 8);
      *reinterpret_cast<u32x4*>(k_lds2[buf] + r * KROW + 8 * v) = xk[u];
    }
#pragma unroll
    for (int u = 0; u < VB; ++u) {
      const int i = tid + 256 * u;
      const int r = i / (VD / 8), v = i % (VD / 8);
      *reinterpret_cast<u32x4*>(v_lds2[buf] + r * VROW + 8 * v) = xv[u];
    }
  };
  // One barrier per tile.  At the top of step `it`: tile `it` is in LDS buffer it & 1, tile it + 1
  // in the staging registers, the rows of tile it + 2 in rows_lds[it & 1], and threads 0 .. 63 hold
  // the block ids of tile it + 3 (whose rows go to rows_lds[(it + 1) & 1] during the step).
  int blk_next = -1;
  if (tid < kKeys) {
    store_row(0, load_block(0), 0);
    store_row(kKeys, load_block(kKeys), 1);
  }
  __syncthreads();
  fetch(0);
  land(0);
  fetch(1);
  __syncthreads();                                     // rows_lds[0] is read: tile 2's rows may go there
  if (tid < kKeys) {
    store_row(2 * kKeys, load_block(2 * kKeys), 0);
    blk_next = load_block(3 * kKeys);
  }
  __syncthreads();
  int it = 0;
  for (int u0 = 0; u0 < total; u0 += kKeys, ++it) {
    const T* k_lds = k_lds2[it & 1];
    const T* v_lds = v_lds2[it & 1];
    // a tile with kept tokens ahead of the window concerns every row; of the others, a tile whose
    // keys lie past this wave's last row, or before its first row's window (and are not kept ones),
    // is none of its business
    const bool kept_tile = u0 < nk;
    const int j0 = u0 - nk + j_lo;            // the tile's first key when it holds window keys only
    if (active && (kept_tile || (j0 <= p0 + nq - 1 &&
                                 !(window > 0 && j0 + kKeys - 1 < p0 - window + 1 && j0 >= keep_first)))) {
      f32x16 st[2];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
        for (int i = 0; i < 16; ++i) st[kb][i] = 0.f;
#pragma unroll
        for (int ks = 0; ks < D / 16; ++ks) {
          const u32x4 a = *reinterpret_cast<const u32x4*>(k_lds + (32 * kb + c) * KROW + 16 * ks + 8 * hf);
          st[kb] = M::run(a, qf[ks], st[kb]);
        }
      }
      // every key of the tile visible to every row of the wave: no masks
      const bool full = !kept_tile && j0 + kKeys - 1 <= p0 && nq == kTile &&
                        (window <= 0 || p0 + kTile - 1 - j0 < window);
      float mt = -INFINITY;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          float v = st[kb][i] * scale2;
          if (softcap > 0.f) v = cap_score_fast(st[kb][i] * scale, cap2, cap_arg);
          if (!full) {
            const int j = key_of(u0 + 32 * kb + (i & 3) + 8 * (i >> 2) + 4 * hf);
            const int dist = pq - j;
            const bool ok = c < nq && dist >= 0 && (window <= 0 || dist < window || j < keep_first);
            v = ok ? v : -INFINITY;
          }
          st[kb][i] = v;
          mt = fmaxf(mt, v);
        }
      mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
      const float m_new = fmaxf(m, mt);
      const bool none = m_new == -INFINITY;
      const float corr = none ? 1.f : __builtin_amdgcn_exp2f(m - m_new);
      float psum = 0.f;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const float pv = none ? 0.f : __builtin_amdgcn_exp2f(st[kb][i] - m_new);
          st[kb][i] = pv;
          psum += pv;
        }
      l = l * corr + psum;          // this lane's keys; the partner's half is added at the end
      m = m_new;
      if (__any(corr != 1.f)) {     // the running max of some row moved
#pragma unroll
        for (int n = 0; n < VB; ++n)
#pragma unroll
          for (int i = 0; i < 16; ++i) o[n][i] *= corr;
      }
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          u32x4 pb;
#pragma unroll
          for (int e = 0; e < 4; ++e) pb[e] = pack2<S>(st[kb][8 * s2 + 2 * e], st[kb][8 * s2 + 2 * e + 1]);
          // transposing read of the row-major tile: a group of 16 lanes reads 4 keys x 16 dims, 8
          // bytes per lane (key i16 >> 2, dims 4 (i16 & 3) .. + 3), and every lane receives the four
          // keys of dim i16 of the group
          const int i16 = c & 15;
          const T* src = v_lds + (32 * kb + 16 * s2 + 4 * hf + (i16 >> 2)) * VROW + 16 * (c >> 4) + 4 * (i16 & 3);
#pragma unroll
          for (int n = 0; n < VB; ++n) {
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4)(src + 32 * n));
            const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4)(src + 32 * n + 8 * VROW));
            const u32x2 lo2 = __builtin_bit_cast(u32x2, lo), hi2 = __builtin_bit_cast(u32x2, hi);
            const u32x4 a = {lo2[0], lo2[1], hi2[0], hi2[1]};
            o[n] = M::run(a, pb, o[n]);
          }
        }
    }
    if (u0 + kKeys < total) land((it + 1) & 1);                // tile it + 1, fetched a step ago
    if (u0 + 2 * kKeys < total) fetch(it & 1);                 // tile it + 2 on its way
    if (tid < kKeys && u0 + 3 * kKeys < total) {
      // rows of tile it + 3 into the buffer the step before read tile it + 1's from
      store_row(u0 + 3 * kKeys, blk_next, (it + 1) & 1);
      blk_next = load_block(u0 + 4 * kKeys);
    }
    __syncthreads();
  }
  if (!active) return;
  l += __shfl_xor(l, 32, 64);
  if (c >= nq) return;
  const float inv = 1.f / l;
#pragma unroll
  for (int n = 0; n < VB; ++n)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[n][i] *= inv;
  if (out_inv_freq != nullptr) turn_back<VB>(o, hf, (float)pq, out_inv_freq, interleaved);
  float gv = 1.f;
  if (gate != nullptr) gv = 1.f / (1.f + expf(-S::to_f32(gate[(int64_t)(t0 + c) * gate_stride + h])));
#pragma unroll
  for (int n = 0; n < VB; ++n)
#pragma unroll
    for (int i = 0; i < 16; ++i)
      out[(int64_t)(t0 + c) * out_stride + (int64_t)h * VD + out_dim(n, i, hf)] = S::from_f32(o[n][i] * gv);
}

// kv_attention_heads_kernel<S, DB, VB>: single rows (decode steps).  One workgroup per (row, KV
// head, chunk of up to 32 of its query heads): the 32 columns of the products hold the chunk's
// query heads, so each key and value byte is read once per KV head whatever the group size.  The
// kRowWaves waves split the window's tiles (wave w takes tiles w, w + kRowWaves, ...), each with
// its own key and value tiles in LDS and its own running max / sum / output, merged at the end.
constexpr int kRowWaves = 8;

template <class S, int DB, int VB>
__global__ __launch_bounds__(64 * kRowWaves) void kv_attention_heads_kernel(
    typename S::T* __restrict__ out, int64_t out_stride, const typename S::T* __restrict__ q,
    int64_t q_stride, const typename S::T* __restrict__ gate, int64_t gate_stride,
    const typename S::T* __restrict__ key_cache, const typename S::T* __restrict__ value_cache,
    const int* __restrict__ block_tables, int max_blocks, const int* __restrict__ token_seq,
    const int64_t* __restrict__ positions, const float* __restrict__ out_inv_freq, int interleaved,
    int heads, int kv_heads, int block_size, int num_blocks, int window, float scale,
    int merge_heads, int keep_first, float softcap) {
  using T = typename S::T;
  using M = Mfma8<S>;
  constexpr int D = 32 * DB, VD = 32 * VB;
  constexpr int KROW = D + 4, VROW = VD + 4;
  constexpr int WAVE_ELEMS = kTile * (KROW + VROW);       // one wave's two tiles, in elements
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int hf = lane >> 5, c = lane & 31;
  T* k_lds = reinterpret_cast<T*>(smem) + (size_t)w * WAVE_ELEMS;
  T* v_lds = k_lds + kTile * KROW;
  const int t = blockIdx.x;
  const int group = heads / kv_heads;
  const int chunks = (group + 31) / 32;
  const int g = blockIdx.y / chunks;
  const int h0 = g * group + (blockIdx.y % chunks) * 32;
  const int nh = min(32, g * group + group - h0);
  const int p = (int)positions[t];
  const int* table = block_tables + (int64_t)token_seq[t] * max_blocks;
  const int lo = window > 0 ? max(0, p - window + 1) : 0;
  const int nk = min(keep_first, lo);         // kept keys ahead of the window
  const int total = nk + p - lo + 1;
  const float cap_arg = softcap > 0.f ? 2.f * 1.4426950408889634f / softcap : 0.f;
  const bool live = c < nh;
  u32x2 qf[D / 8];
#pragma unroll
  for (int ks = 0; ks < D / 8; ++ks) {
    u32x2 v = {0u, 0u};
    if (live)
      v = *reinterpret_cast<const u32x2*>(q + (int64_t)t * q_stride + (int64_t)(h0 + c) * D + 8 * ks + 4 * hf);
    qf[ks] = v;
  }
  f32x16 o[VB];
#pragma unroll
  for (int n = 0; n < VB; ++n)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[n][i] = 0.f;
  float m = -INFINITY, l = 0.f;

  // A wave's share of a tile is D / 8 + VD / 8 pieces of 8 bytes per lane, all issued before any
  // is used and one tile ahead.  Lanes 0..31 look the 32 tokens of the tile up once and hand the
  // row numbers round with shuffles.
  constexpr int KP = D / 8, VP = VD / 8;
  u32x2 xk[KP], xv[VP];
  auto fetch = [&](int u0) {
    const int ur = u0 + c;
    long long row = -1;
    if (ur < total) {
      const int jr = ur < nk ? ur : ur - nk + lo;
      int blk = table[jr / block_size];
      blk = (unsigned)blk < (unsigned)num_blocks ? blk : 0;
      row = ((long long)blk * block_size + jr % block_size) * kv_heads + g;
    }
#pragma unroll
    for (int u = 0; u < KP; ++u) {
      const int i = lane + kWave * u;
      const int r = i / (D / 4), v = i % (D / 4);
      const long long rb = __shfl(row, r, 64);
      const u32x2 got = *reinterpret_cast<const u32x2*>(key_cache + (rb >= 0 ? rb * D + 4 * v : 0));
      xk[u] = rb >= 0 ? got : u32x2{0u, 0u};
    }
#pragma unroll
    for (int u = 0; u < VP; ++u) {
      const int i = lane + kWave * u;
      const int r = i / (VD / 4), v = i % (VD / 4);
      const long long rb = __shfl(row, r, 64);
      const u32x2 got = *reinterpret_cast<const u32x2*>(value_cache + (rb >= 0 ? rb * VD + 4 * v : 0));
      xv[u] = rb >= 0 ? got : u32x2{0u, 0u};
    }
  };
  fetch(w * kTile);
  for (int u0 = w * kTile; u0 < total; u0 += kRowWaves * kTile) {
#pragma unroll
    for (int u = 0; u < KP; ++u) {
      const int i = lane + kWave * u;
      const int r = i / (D / 4), v = i % (D / 4);
      *reinterpret_cast<u32x2*>(k_lds + r * KROW + 4 * v) = xk[u];
    }
#pragma unroll
    for (int u = 0; u < VP; ++u) {
      const int i = lane + kWave * u;
      const int r = i / (VD / 4), v = i % (VD / 4);
      *reinterpret_cast<u32x2*>(v_lds + r * VROW + 4 * v) = xv[u];
    }
    if (u0 + kRowWaves * kTile < total) fetch(u0 + kRowWaves * kTile);
    wave_sync();
    f32x16 st;
#pragma unroll
    for (int i = 0; i < 16; ++i) st[i] = 0.f;
#pragma unroll
    for (int ks = 0; ks < D / 8; ++ks) {
      const u32x2 a = *reinterpret_cast<const u32x2*>(k_lds + c * KROW + 8 * ks + 4 * hf);
      st = M::run(a, qf[ks], st);
    }
    float mt = -INFINITY;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int u = u0 + (i & 3) + 8 * (i >> 2) + 4 * hf;
      float v = st[i] * scale;
      if (softcap > 0.f) v = cap_score_fast(v, softcap, cap_arg);
      st[i] = (live && u < total) ? v : -INFINITY;
      mt = fmaxf(mt, st[i]);
    }
    mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
    const float m_new = fmaxf(m, mt);
    const float corr = m_new == -INFINITY ? 1.f : expf(m - m_new);
    float psum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      st[i] = m_new == -INFINITY ? 0.f : expf(st[i] - m_new);
      psum += st[i];
    }
    l = l * corr + psum;
    m = m_new;
#pragma unroll
    for (int n = 0; n < VB; ++n)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[n][i] *= corr;
#pragma unroll
    for (int s8 = 0; s8 < 4; ++s8) {
      uint32_t hb[4], lb[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float pv = st[4 * s8 + e];
        hb[e] = bits16<S>(pv);
        lb[e] = bits16<S>(pv - from_bits16<S>(hb[e]));
      }
      const u32x2 hi = {hb[0] | (hb[1] << 16), hb[2] | (hb[3] << 16)};
      const u32x2 lo2 = {lb[0] | (lb[1] << 16), lb[2] | (lb[3] << 16)};
#pragma unroll
      for (int n = 0; n < VB; ++n) {
        // V^T operand from the row-major tile: value dim 32 n + c of keys 8 s8 + 4 hf .. + 3
        const uint16_t* col = reinterpret_cast<const uint16_t*>(v_lds) + (8 * s8 + 4 * hf) * VROW + 32 * n + c;
        const u32x2 a = {(uint32_t)col[0] | ((uint32_t)col[VROW] << 16),
                         (uint32_t)col[2 * VROW] | ((uint32_t)col[3 * VROW] << 16)};
        o[n] = M::run(a, hi, o[n]);
        o[n] = M::run(a, lo2, o[n]);
      }
    }
    wave_sync();
  }
  l += __shfl_xor(l, 32, 64);
  // merge the waves through LDS (the tiles are done with): [wave][head][2 + VD]
  __syncthreads();
  float* merge = reinterpret_cast<float*>(smem);
  if (live) {
    float* mine = merge + ((size_t)w * merge_heads + c) * (2 + VD);
    if (hf == 0) {
      mine[0] = m;
      mine[1] = l;
    }
#pragma unroll
    for (int n = 0; n < VB; ++n)
#pragma unroll
      for (int i = 0; i < 16; ++i) mine[2 + out_dim(n, i, hf)] = o[n][i];
  }
  __syncthreads();
  auto merged = [&](int hh, int d) {
    float mm = -INFINITY;
    for (int ww = 0; ww < kRowWaves; ++ww) mm = fmaxf(mm, merge[((size_t)ww * merge_heads + hh) * (2 + VD)]);
    float ll = 0.f, ov = 0.f;
    for (int ww = 0; ww < kRowWaves; ++ww) {
      const float* src = merge + ((size_t)ww * merge_heads + hh) * (2 + VD);
      const float f = src[0] == -INFINITY ? 0.f : expf(src[0] - mm);
      ll += src[1] * f;
      ov += src[2 + d] * f;
    }
    return ov / ll;
  };
  for (int i = tid; i < nh * VD; i += 64 * kRowWaves) {
    const int hh = i / VD, d = i - hh * VD;
    float val = merged(hh, d);
    if (out_inv_freq != nullptr) {
      const bool is_a = interleaved ? (d & 1) == 0 : d < VD / 2;
      const int other = interleaved ? (d ^ 1) : (is_a ? d + VD / 2 : d - VD / 2);
      const int f = interleaved ? d >> 1 : (is_a ? d : d - VD / 2);
      float s, c2;
      sincosf((float)p * out_inv_freq[f], &s, &c2);
      const float ov = merged(hh, other);
      val = is_a ? val * c2 + ov * s : val * c2 - ov * s;
    }
    if (gate != nullptr) val *= 1.f / (1.f + expf(-S::to_f32(gate[(int64_t)t * gate_stride + h0 + hh])));
    out[(int64_t)t * out_stride + (int64_t)(h0 + hh) * VD + d] = S::from_f32(val);
  }
}

template <class S, int DB, int VB>
int launch_heads_one(dim3 grid, hipStream_t stream, typename S::T* out, int64_t out_stride,
                     const typename S::T* q, int64_t q_stride, const typename S::T* gate,
                     int64_t gate_stride, const typename S::T* key_cache,
                     const typename S::T* value_cache, const int* block_tables, int max_blocks,
                     const int* token_seq, const int64_t* positions, const float* out_inv_freq,
                     int interleaved, int heads, int kv_heads, int block_size, int num_blocks,
                     int window, float scale, int keep_first, float softcap) {
  constexpr int D = 32 * DB, VD = 32 * VB;
  const int group = heads / kv_heads;
  const int merge_heads = group < 32 ? group : 32;
  const size_t tiles = (size_t)kRowWaves * kTile * (D + 4 + VD + 4) * sizeof(typename S::T);
  const size_t merge = (size_t)kRowWaves * merge_heads * (2 + VD) * sizeof(float);
  const size_t lds = tiles > merge ? tiles : merge;
  if (lds > 160 * 1024) return VLA_ERR_HEAD_SIZE;
  static std::atomic<size_t> allowed{64 * 1024};   // raised once per kernel, not per launch
  if (lds > allowed.load(std::memory_order_relaxed)) {
    VLA_SEQ_HIP_CHECK(hipFuncSetAttribute(
        reinterpret_cast<const void*>(&kv_attention_heads_kernel<S, DB, VB>),
        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    allowed.store(lds, std::memory_order_relaxed);
  }
  kv_attention_heads_kernel<S, DB, VB><<<grid, 64 * kRowWaves, lds, stream>>>(
      out, out_stride, q, q_stride, gate, gate_stride, key_cache, value_cache, block_tables,
      max_blocks, token_seq, positions, out_inv_freq, interleaved, heads, kv_heads, block_size,
      num_blocks, window, scale, merge_heads, keep_first, softcap);
  VLA_SEQ_HIP_CHECK(hipGetLastError());
  return VLA_OK;
}

template <class S, int DB, int VB>
int launch_tiles_one(dim3 grid, hipStream_t stream, typename S::T* out, int64_t out_stride,
                     const typename S::T* q, int64_t q_stride, const typename S::T* gate,
                     int64_t gate_stride, const typename S::T* key_cache,
                     const typename S::T* value_cache, const int* block_tables, int max_blocks,
                     const int* qsl, const int* ctx, const float* out_inv_freq, int interleaved,
                     int heads, int kv_heads, int block_size, int num_blocks, int window,
                     float scale, int head_waves, int keep_first, float softcap) {
  kv_attention_tile_kernel<S, DB, VB><<<grid, 256, 0, stream>>>(
      out, out_stride, q, q_stride, gate, gate_stride, key_cache, value_cache, block_tables,
      max_blocks, qsl, ctx, out_inv_freq, interleaved, heads, kv_heads, block_size, num_blocks,
      window, scale, head_waves, keep_first, softcap);
  VLA_SEQ_HIP_CHECK(hipGetLastError());
  return VLA_OK;
}

// dim / 32 and vdim / 32 in 1 .. 4 -> the instantiation
#define VLA_KV_BY_SIZE(FN, S, db, vb, ...)                         \
  switch ((db) * 4 + (vb)-5) {                                     \
    case 0: return FN<S, 1, 1>(__VA_ARGS__);                       \
    case 1: return FN<S, 1, 2>(__VA_ARGS__);                       \
    case 2: return FN<S, 1, 3>(__VA_ARGS__);                       \
    case 3: return FN<S, 1, 4>(__VA_ARGS__);                       \
    case 4: return FN<S, 2, 1>(__VA_ARGS__);                       \
    case 5: return FN<S, 2, 2>(__VA_ARGS__);                       \
    case 6: return FN<S, 2, 3>(__VA_ARGS__);                       \
    case 7: return FN<S, 2, 4>(__VA_ARGS__);                       \
    case 8: return FN<S, 3, 1>(__VA_ARGS__);                       \
    case 9: return FN<S, 3, 2>(__VA_ARGS__);                       \
    case 10: return FN<S, 3, 3>(__VA_ARGS__);                      \
    case 11: return FN<S, 3, 4>(__VA_ARGS__);                      \
    case 12: return FN<S, 4, 1>(__VA_ARGS__);                      \
    case 13: return FN<S, 4, 2>(__VA_ARGS__);                      \
    case 14: return FN<S, 4, 3>(__VA_ARGS__);                      \
    case 15: return FN<S, 4, 4>(__VA_ARGS__);                      \
    default: return VLA_ERR_HEAD_SIZE;                             \
  }

template <class S, class... A>
int launch_heads(int db, int vb, A... a) {
  VLA_KV_BY_SIZE(launch_heads_one, S, db, vb, a...)
}
template <class S, class... A>
int launch_tiles(int db, int vb, A... a) {
  VLA_KV_BY_SIZE(launch_tiles_one, S, db, vb, a...)
}

bool mfma_sizes(int dim, int vdim) {
  return dim % 32 == 0 && dim >= 32 && dim <= 128 && vdim % 32 == 0 && vdim >= 32 && vdim <= 128;
}

}  // namespace
}  // namespace seq
}  // namespace vla

using namespace vla;
using namespace vla::seq;

extern "C" int vla_seq_rotary_kv_write(void* q, int64_t q_stride, const void* k, int64_t k_stride,
                                       const void* v, int64_t v_stride, void* key_cache,
                                       void* value_cache, const int64_t* positions,
                                       const int64_t* slot_mapping, const float* inv_freq,
                                       const float* value_inv_freq, int num_tokens, int heads,
                                       int kv_heads, int dim, int vdim, int rot_dims,
                                       int interleaved, int block_size, int num_blocks, int dtype,
                                       const float* q_norm, const float* k_norm, float norm_eps,
                                       const void* v_other, int64_t v_other_stride,
                                       const float* v_blend, void* stream) {
  if (num_tokens == 0) return VLA_OK;
  if (!q || !k || !v || !key_cache || !value_cache || !positions || !slot_mapping || num_tokens < 0 ||
      heads <= 0 || kv_heads <= 0 || dim <= 0 || vdim <= 0 || rot_dims < 0 || rot_dims > dim ||
      (rot_dims & 1) || (rot_dims > 0 && !inv_freq) || block_size <= 0 || num_blocks <= 0 ||
      q_stride < (int64_t)heads * dim || k_stride < (int64_t)kv_heads * dim ||
      v_stride < (int64_t)kv_heads * vdim ||
      (v_other && (!v_blend || value_inv_freq || v_other_stride < (int64_t)kv_heads * vdim)))
    return VLA_ERR_ARG;
  return with_dtype(dtype, [&](auto s) {
    using S = decltype(s);
    using T = typename S::T;
    rotary_kv_write_kernel<S><<<num_tokens, 256, 0, (hipStream_t)stream>>>(
        (T*)q, q_stride, (const T*)k, k_stride, (const T*)v, v_stride, (T*)key_cache,
        (T*)value_cache, positions, slot_mapping, inv_freq, value_inv_freq, heads, kv_heads, dim,
        vdim, rot_dims, interleaved, (int64_t)num_blocks * block_size, q_norm, k_norm, norm_eps,
        (const T*)v_other, v_other_stride, v_blend);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}

extern "C" int vla_seq_kv_attention(void* out, int64_t out_stride, const void* q, int64_t q_stride,
                                    const void* gate, int64_t gate_stride, const void* key_cache,
                                    const void* value_cache, const int* block_tables,
                                    int max_blocks, const int* token_seq, const int64_t* positions,
                                    const float* out_inv_freq, int interleaved, int num_tokens,
                                    int heads, int kv_heads, int dim, int vdim, int block_size,
                                    int num_blocks, int window, float scale, int dtype,
                                    int keep_first, float softcap, void* stream) {
  if (num_tokens == 0) return VLA_OK;
  if (!out || !q || !key_cache || !value_cache || !block_tables || !token_seq || !positions ||
      num_tokens < 0 || heads <= 0 || kv_heads <= 0 || heads % kv_heads != 0 || block_size <= 0 ||
      num_blocks <= 0 || max_blocks <= 0 || out_stride < (int64_t)heads * vdim ||
      q_stride < (int64_t)heads * dim || (gate && gate_stride < heads) || keep_first < 0 ||
      !(softcap >= 0.f))
    return VLA_ERR_ARG;
  if (dim <= 0 || dim > kMaxDim || vdim <= 0 || vdim > kMaxDim) return VLA_ERR_HEAD_SIZE;
  return with_dtype(dtype, [&](auto s) {
    using S = decltype(s);
    using T = typename S::T;
    if constexpr (sizeof(T) == 2) {
      // 16-bit rows on the matrix cores when the head sizes and the alignment allow
      if (g_kv_kernel.load(std::memory_order_relaxed) == 0 && mfma_sizes(dim, vdim) &&
          ((uintptr_t)q % 8) == 0 && ((q_stride * 2) % 8) == 0 && ((uintptr_t)key_cache % 8) == 0 &&
          ((uintptr_t)value_cache % 8) == 0) {
        const int group = heads / kv_heads;
        const dim3 grid(num_tokens, kv_heads * ((group + 31) / 32));
        const int rc = launch_heads<S>(dim / 32, vdim / 32, grid, (hipStream_t)stream, (T*)out, out_stride,
                                       (const T*)q, q_stride, (const T*)gate, gate_stride,
                                       (const T*)key_cache, (const T*)value_cache, block_tables,
                                       max_blocks, token_seq, positions, out_inv_freq, interleaved,
                                       heads, kv_heads, block_size, num_blocks, window, scale,
                                       window > 0 ? keep_first : 0, softcap);
        if (rc != VLA_ERR_HEAD_SIZE) return rc;
      }
    }
    const dim3 grid(num_tokens, (heads + kHeadsPerGroup - 1) / kHeadsPerGroup);
    kv_attention_kernel<S><<<grid, kWave * kHeadsPerGroup, 0, (hipStream_t)stream>>>(
        (T*)out, out_stride, (const T*)q, q_stride, (const T*)gate, gate_stride,
        (const T*)key_cache, (const T*)value_cache, block_tables, max_blocks, token_seq, positions,
        out_inv_freq, interleaved, heads, kv_heads, dim, vdim, block_size, num_blocks, window, scale,
        window > 0 ? keep_first : 0, softcap);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}

// 0: pick per shape; 1: always the one-wave-per-(row, head) kernel (tests run both)
extern "C" int vla_seq_set_kv_attention_kernel(int mode) {
  if (mode < 0 || mode > 1) return VLA_ERR_ARG;
  g_kv_kernel.store(mode, std::memory_order_relaxed);
  return VLA_OK;
}

extern "C" int vla_seq_kv_attention_tiles_supported(int dim, int vdim, int dtype) {
  return (dtype == VLA_F16 || dtype == VLA_BF16) && mfma_sizes(dim, vdim) &&
         g_kv_kernel.load(std::memory_order_relaxed) == 0;
}

extern "C" int vla_seq_kv_attention_tiles(
    void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* gate,
    int64_t gate_stride, const void* key_cache, const void* value_cache, const int* block_tables,
    int max_blocks, const int* query_start_loc, const int* context_lens, const float* out_inv_freq,
    int interleaved, int num_seqs, int max_query_len, int heads, int kv_heads, int dim, int vdim,
    int block_size, int num_blocks, int window, float scale, int dtype, int keep_first,
    float softcap, void* stream) {
  if (num_seqs == 0 || max_query_len == 0) return VLA_OK;
  if (keep_first < 0 || !(softcap >= 0.f)) return VLA_ERR_ARG;
  if (window <= 0) keep_first = 0;
  if (!out || !q || !key_cache || !value_cache || !block_tables || !query_start_loc || !context_lens ||
      num_seqs < 0 || num_seqs > 65535 || max_query_len < 0 || heads <= 0 || kv_heads <= 0 ||
      heads % kv_heads != 0 || block_size <= 0 || num_blocks <= 0 || max_blocks <= 0 ||
      out_stride < (int64_t)heads * vdim || q_stride < (int64_t)heads * dim ||
      (gate && gate_stride < heads))
    return VLA_ERR_ARG;
  if ((dtype != VLA_F16 && dtype != VLA_BF16) || !mfma_sizes(dim, vdim)) return VLA_ERR_HEAD_SIZE;
  // 8-byte fragment loads: query rows and cache rows must allow them
  if (((uintptr_t)q % 8) || ((q_stride * 2) % 8) || ((uintptr_t)key_cache % 8) ||
      ((uintptr_t)value_cache % 8))
    return VLA_ERR_ARG;
  // 16-byte fragment loads: query rows and cache rows must allow them
  if (((uintptr_t)q % 16) || ((q_stride * 2) % 16) || ((uintptr_t)key_cache % 16) ||
      ((uintptr_t)value_cache % 16))
    return VLA_ERR_ARG;
  const int group = heads / kv_heads;
  const int head_waves = group >= 3 ? 4 : group;      // waves of a workgroup that are heads
  const int tile_rows = kTile * (4 / head_waves);
  const dim3 grid((max_query_len + tile_rows - 1) / tile_rows,
                  kv_heads * ((group + head_waves - 1) / head_waves), num_seqs);
  if (dtype == VLA_BF16)
    return launch_tiles<BF16>(dim / 32, vdim / 32, grid, (hipStream_t)stream, (__bf16*)out, out_stride,
                              (const __bf16*)q, q_stride, (const __bf16*)gate, gate_stride,
                              (const __bf16*)key_cache, (const __bf16*)value_cache, block_tables,
                              max_blocks, query_start_loc, context_lens, out_inv_freq, interleaved,
                              heads, kv_heads, block_size, num_blocks, window, scale, head_waves,
                              keep_first, softcap);
  return launch_tiles<F16>(dim / 32, vdim / 32, grid, (hipStream_t)stream, (_Float16*)out, out_stride,
                           (const _Float16*)q, q_stride, (const _Float16*)gate, gate_stride,
                           (const _Float16*)key_cache, (const _Float16*)value_cache, block_tables,
                           max_blocks, query_start_loc, context_lens, out_inv_freq, interleaved, heads,
                           kv_heads, block_size, num_blocks, window, scale, head_waves, keep_first,
                           softcap);
}
