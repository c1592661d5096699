// Causal softmax attention whose keys and values are up-projections of one cached latent per token.
//
// Per token the cache holds one row [latent (rank) | shared rotated key part (rot)] in the model
// dtype: cache [num_blocks, block_size, rank + rot].  Head h's key is [W_uk,h c | k_rot] and its
// value W_uv,h c, so with q_lat,h = W_uk,h^T q_plain,h (the caller's matrix product)
//   score = (q_lat,h . c + q_rot,h . k_rot) * scale,    o_lat,h = sum_j p_j c_j,
// and the head's output is W_uv,h o_lat,h (the caller's product again): every head reads the same
// rows, nothing per head is cached.  latent_rotary_write norms the step's latents, rotates the
// shared key part and the queries' rotated parts (pairs (2i, 2i + 1) or (i, i + rot_dims / 2),
// frequencies from a table, sine and cosine times a magnitude), and writes the cache rows; the
// attention kernels then read every query row's keys from the cache, so prompts, portions of
// prompts and decode steps are one case.  An optional window keeps 0 <= p - j < window; an optional
// gate multiplies a head's sums by the sigmoid of one number per (token, head) (the head's
// up-projection that follows is linear, so the gate may stand on either side of it).  Angles, norms,
// scores, softmax and the weighted sum are fp32.
//
// latent_attention_kernel: one wave per (token, head), any dtype, rank up to 1024.  A tile is 64
// keys: lane j scores key j against the query held in LDS, the wave reduces max / sum (online
// softmax across tiles), then lane d accumulates sum_j p_j c_j[d] with coalesced reads.
#include <atomic>

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
    int heads, int rank, int rot, int rot_dims, int64_t num_slots, int interleaved) {
  using T = typename S::T;
  __shared__ float red[16];
  const int t = blockIdx.x;
  const float p = (float)positions[t];
  const int half = rot_dims / 2;        // pairs that turn; what follows them passes unchanged
  const int first_mul = interleaved ? 2 : 1, second = interleaved ? 1 : half;   // pair f: f * first_mul, + second
  T* qr = q + (int64_t)t * q_stride + q_first;
  for (int i = threadIdx.x; i < heads * half; i += blockDim.x) {
    const int h = i / half, f = i - h * half;
    T* e = qr + (int64_t)h * q_head_stride + first_mul * f;
    float a = S::to_f32(e[0]), b = S::to_f32(e[second]);
    turn_scaled(a, b, p * inv_freq[f], magnitude);
    e[0] = S::from_f32(a);
    e[second] = S::from_f32(b);
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
    float a = S::to_f32(kr[rank + first_mul * f]), b = S::to_f32(kr[rank + first_mul * f + second]);
    turn_scaled(a, b, p * inv_freq[f], magnitude);
    row[rank + first_mul * f] = S::from_f32(a);
    row[rank + first_mul * f + second] = S::from_f32(b);
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
    int heads, int rank, int rot, int block_size, int num_blocks, float scale, int window,
    const typename S::T* __restrict__ gate, int64_t gate_stride) {
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
  const int lo = window > 0 ? max(0, p - window + 1) : 0;
  for (int j0 = lo; j0 <= p; j0 += kWave) {
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
  float inv = 1.f / l;
  if (gate != nullptr) inv /= 1.f + expf(-S::to_f32(gate[(int64_t)t * gate_stride + h]));
  typename S::T* orow = out + (int64_t)t * out_token_stride + (int64_t)h * out_head_stride;
#pragma unroll
  for (int c = 0; c < kAccum; ++c) {
    const int d = lane + c * kWave;
    if (d < rank) orow[d] = S::from_f32(acc[c] * inv);
  }
}


// ---------------------------------------------------------------------------------------------
// latent_attention_tile_kernel<S, VBW>: 16-bit models on 32x32x16 MFMAs, prompts, portions and
// decode steps alike.  Every head reads the same cache rows, so a workgroup takes 32 query rows
// that are (token, head) pairs of one sequence -- up to 32 heads of one token, or all heads of
// 32 / heads consecutive tokens -- and walks the keys from the first to the last row's position in
// tiles of 32, staged through LDS once for its four waves (loaded one tile ahead into registers; the
// rows' places in the paged cache are looked up two tiles ahead).  One tile and the partial scores
// are all the LDS a workgroup holds, so two workgroups share a CU.  Both products run in transposed form, lane =
// (hf, c) = (lane >> 5, lane & 31):
//   S^T = K q^T   A = K    lane: key c, dims 16 ks + 8 hf .. + 7       (LDS, 16 bytes)
//                 B = q^T  lane: query row c, the same dims           (registers, loaded once)
//                 C        lane: query row c, keys (i & 3) + 8 (i >> 2) + 4 hf, i = 0 .. 15
//   O^T = C^T P^T B = P^T  lane: query row c, registers 8 s .. 8 s + 7 of C
//                 A = C^T  lane: latent dim 32 n + c of the same eight keys (two transposing reads
//                          of the row-major tile: the latent is key and value at once)
// The four waves split the first product's k-steps (rank + rot dims) and add their partial scores
// through LDS, so each holds the whole 32 x 32 score block and the same running max and sum; they
// split the second product's blocks of 32 latent dims (wave w owns blocks w, w + 4, ...).  Scores,
// max / sum (base 2) and accumulators are fp32; a weight enters the second product rounded to the
// model dtype.  With key_splits > 1 (steps of short runs over long contexts) the keys of a row tile
// are shared out to that many workgroups, which leave their sums in scratch for a merge launch.
template <class S>
struct LatentMfma;
template <>
struct LatentMfma<BF16> {
  static __device__ __forceinline__ f32x16 run(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b),
                                                   c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack2(float a, float b) {
    const f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
  }
};
template <>
struct LatentMfma<F16> {
  static __device__ __forceinline__ f32x16 run(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c,
                                                  0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack2(float a, float b) {
    const f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
  }
};

constexpr int kTileKeys = 32;
constexpr int kTileRows = 32;
typedef short lat_s16x4 __attribute__((ext_vector_type(4)));
typedef lat_s16x4 __attribute__((address_space(3))) * lat_lds_s16x4;

template <class S, int VBW>
__global__ __launch_bounds__(256) void latent_attention_tile_kernel(
    typename S::T* __restrict__ out, int64_t out_token_stride, int64_t out_head_stride,
    LatentQuery<S> q, const typename S::T* __restrict__ cache, const int* __restrict__ block_tables,
    int max_blocks, const int* __restrict__ query_start_loc, const int* __restrict__ context_lens,
    int heads, int rank, int rot, int block_size, int num_blocks, float scale, int hb, int tb,
    int key_splits, float* __restrict__ part_o, float* __restrict__ part_ml, int num_tokens,
    int window, const typename S::T* __restrict__ gate, int64_t gate_stride) {
  using T = typename S::T;
  using M = LatentMfma<S>;
  constexpr int WP = 2 * VBW + 2;                      // 16-byte pieces of a tile a thread stages
  extern __shared__ __align__(16) unsigned char smem[];
  const int width = rank + rot, row_elems = width + 8;   // rows stay 16-byte aligned
  const int row_pieces = width / 8, tile_pieces = kTileKeys * row_pieces;
  T* k_lds = reinterpret_cast<T*>(smem);                                     // [32][row_elems]
  float* s_lds = reinterpret_cast<float*>(k_lds + kTileKeys * row_elems);    // [4][4][64][4]
  long long* rows_lds = reinterpret_cast<long long*>(s_lds + 4 * 16 * 64);   // [2][32]
  const int b = blockIdx.z;
  // the last tiles of a run have the most keys to walk: they are dispatched first
  const int flat_x = gridDim.x - 1 - blockIdx.x;
  const int tile_x = flat_x / key_splits, split = flat_x - tile_x * key_splits;
  const int run = query_start_loc[b + 1] - query_start_loc[b];
  const int tq0 = tile_x * tb;
  if (tq0 >= run) return;
  const int ntok = min(tb, run - tq0);
  const int h0 = blockIdx.y * hb, nh = min(hb, heads - h0);
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int hf = lane >> 5, c = lane & 31;
  const int t_first = query_start_loc[b] + tq0;
  const int p_first = context_lens[b] + tq0, p_end = p_first + ntok - 1;
  // this workgroup's share of the keys j_first .. p_end (j_first: where the first row's window
  // starts): whole tiles, the last share may be short or empty
  const int j_first = window > 0 ? max(0, p_first - window + 1) : 0;
  const int share = ((p_end - j_first + key_splits) / key_splits + kTileKeys - 1) / kTileKeys * kTileKeys;
  const int j_begin = j_first + split * share;
  const int p_last = min(p_end, j_begin + share - 1);      // the last key this workgroup reads
  const int my_tok = c / hb, my_head = c - my_tok * hb;
  const bool my_row = my_tok < ntok && my_head < nh;
  const bool all_rows = ntok * hb == kTileRows && nh == hb;    // no idle row in this workgroup
  const int pq = p_first + my_tok;
  const int* table = block_tables + (int64_t)b * max_blocks;
  const float scale2 = scale * 1.4426950408889634f;    // scores in base 2

  // the query rows stay in registers: a wave keeps the k-steps w, w + 4, ... of the first product
  const int ksteps = width / 16, vb = rank / 32;
  u32x4 qf[WP];
#pragma unroll
  for (int u = 0; u < WP; ++u) {
    const int d = 16 * (w + 4 * u) + 8 * hf;
    u32x4 val = {0u, 0u, 0u, 0u};
    if (my_row && d < width) {
      const int64_t t = t_first + my_tok, h = h0 + my_head;
      val = d < rank ? *reinterpret_cast<const u32x4*>(q.lat + t * q.lat_token_stride + h * q.lat_head_stride + d)
                     : *reinterpret_cast<const u32x4*>(q.rot + t * q.rot_token_stride + h * q.rot_head_stride + d - rank);
    }
    qf[u] = val;
  }
  f32x16 o[VBW];
#pragma unroll
  for (int n = 0; n < VBW; ++n)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[n][i] = 0.f;
  float m = -INFINITY, l = 0.f;

  // threads 0 .. 31 look the rows of a tile up: the block id is read one step before it is used
  auto load_block = [&](int j0) {
    const int j = j0 + tid;
    int blk = -1;
    if (j <= p_last) {
      blk = table[j / block_size];
      blk = (unsigned)blk < (unsigned)num_blocks ? blk : 0;
    }
    return blk;
  };
  auto store_row = [&](int j0, int blk, int buf) {
    const int j = j0 + tid;
    // the row's first element in the cache, so that a fetch only adds its piece's offset
    rows_lds[buf * kTileKeys + tid] = blk < 0 ? -1 : ((long long)blk * block_size + j % block_size) * width;
  };
  // where this thread's pieces of a tile sit: key row of the tile, offset in the cache row, offset
  // in the LDS tile (the same for every tile, so the divisions are done once)
  u32x4 stage[WP];
  int piece_row[WP], piece_src[WP], piece_dst[WP];
#pragma unroll
  for (int u = 0; u < WP; ++u) {
    const int i = tid + 256 * u;
    const int r = i / row_pieces, v = i - r * row_pieces;
    piece_row[u] = i < tile_pieces ? r : -1;
    piece_src[u] = 8 * v;
    piece_dst[u] = r * row_elems + 8 * v;
  }
  auto fetch = [&](int buf) {
#pragma unroll
    for (int u = 0; u < WP; ++u) {
      u32x4 got = {0u, 0u, 0u, 0u};
      if (piece_row[u] >= 0) {
        const long long row = rows_lds[buf * kTileKeys + piece_row[u]];
        if (row >= 0) got = *reinterpret_cast<const u32x4*>(cache + row + piece_src[u]);
      }
      stage[u] = got;
    }
  };
  auto land = [&]() {
#pragma unroll
    for (int u = 0; u < WP; ++u)
      if (piece_row[u] >= 0)
        *reinterpret_cast<u32x4*>(k_lds + piece_dst[u]) = stage[u];
  };
  // Three barriers per tile (two workgroups share a CU and fill each other's waits).  At the top of
  // step `it`: tile `it` is in LDS, tile it + 1 in the staging registers, the rows of tile it + 2
  // in rows_lds[it & 1], and threads 0 .. 31 hold the block ids of tile it + 3.
  int blk_next = -1;
  if (tid < kTileKeys) {
    store_row(j_begin, load_block(j_begin), 0);
    store_row(j_begin + kTileKeys, load_block(j_begin + kTileKeys), 1);
  }
  __syncthreads();
  fetch(0);
  land();
  fetch(1);
  __syncthreads();
  if (tid < kTileKeys) {
    store_row(j_begin + 2 * kTileKeys, load_block(j_begin + 2 * kTileKeys), 0);
    blk_next = load_block(j_begin + 3 * kTileKeys);
  }
  __syncthreads();
  int it = 0;
  for (int j0 = j_begin; j0 <= p_last; j0 += kTileKeys, ++it) {
    f32x16 st;
#pragma unroll
    for (int i = 0; i < 16; ++i) st[i] = 0.f;
#pragma unroll
    for (int u = 0; u < WP; ++u) {
      const int ks = w + 4 * u;
      if (ks < ksteps) {
        const u32x4 a = *reinterpret_cast<const u32x4*>(k_lds + c * row_elems + 16 * ks + 8 * hf);
        st = M::run(a, qf[u], st);
      }
    }
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      const f32x4 part = {st[4 * i4], st[4 * i4 + 1], st[4 * i4 + 2], st[4 * i4 + 3]};
      *reinterpret_cast<f32x4*>(s_lds + ((w * 4 + i4) * 64 + lane) * 4) = part;
    }
    __syncthreads();
#pragma unroll
    for (int ow = 1; ow < 4; ++ow) {
      const int w2 = (w + ow) & 3;
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const f32x4 part = *reinterpret_cast<const f32x4*>(s_lds + ((w2 * 4 + i4) * 64 + lane) * 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) st[4 * i4 + e] += part[e];
      }
    }
    // (the sum above runs in a different order in each wave; every wave keeps its own max and sum, and
    // they only need to agree with its own weights)
    // every key of the tile visible to every row of a full workgroup: no masks
    const bool full = all_rows && j0 + kTileKeys - 1 <= p_first && (window <= 0 || p_end - j0 < window);
    float mt = -INFINITY;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      float v = st[i] * scale2;
      if (!full) {
        const int j = j0 + (i & 3) + 8 * (i >> 2) + 4 * hf;
        v = my_row && j <= pq && (window <= 0 || pq - j < window) ? v : -INFINITY;
      }
      st[i] = v;
      mt = fmaxf(mt, v);
    }
    mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
    const float m_new = fmaxf(m, mt);
    const bool none = m_new == -INFINITY;
    const float corr = none ? 1.f : __builtin_amdgcn_exp2f(m - m_new);
    float psum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float pv = none ? 0.f : __builtin_amdgcn_exp2f(st[i] - m_new);
      st[i] = pv;
      psum += pv;
    }
    l = l * corr + psum;            // this lane's keys; the partner's half is added at the end
    m = m_new;
    if (__any(corr != 1.f)) {
#pragma unroll
      for (int n = 0; n < VBW; ++n)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[n][i] *= corr;
    }
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2) {
      u32x4 pb;
#pragma unroll
      for (int e = 0; e < 4; ++e) pb[e] = M::pack2(st[8 * s2 + 2 * e], st[8 * s2 + 2 * e + 1]);
      // transposing read of the row-major tile: a group of 16 lanes reads 4 keys x 16 dims, 8
      // bytes per lane, and every lane receives the four keys of one dim of the group
      const int i16 = c & 15;
      const T* src = k_lds + (16 * s2 + 4 * hf + (i16 >> 2)) * row_elems + 16 * (c >> 4) + 4 * (i16 & 3);
#pragma unroll
      for (int n = 0; n < VBW; ++n) {
        const int blk = w + 4 * n;
        if (blk < vb) {
          const lat_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lat_lds_s16x4)(src + 32 * blk));
          const lat_s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lat_lds_s16x4)(src + 32 * blk + 8 * row_elems));
          const u32x2 lo2 = __builtin_bit_cast(u32x2, lo), hi2 = __builtin_bit_cast(u32x2, hi);
          const u32x4 a = {lo2[0], lo2[1], hi2[0], hi2[1]};
          o[n] = M::run(a, pb, o[n]);
        }
      }
    }
    __syncthreads();                                             // everyone is done with tile it
    if (j0 + kTileKeys <= p_last) land();                        // tile it + 1, fetched a step ago
    if (j0 + 2 * kTileKeys <= p_last) fetch(it & 1);             // tile it + 2 on its way
    if (tid < kTileKeys && j0 + 3 * kTileKeys <= p_last) {
      store_row(j0 + 3 * kTileKeys, blk_next, (it + 1) & 1);
      blk_next = load_block(j0 + 4 * kTileKeys);
    }
    __syncthreads();
  }
  l += __shfl_xor(l, 32, 64);
  if (!my_row) return;
  if (key_splits > 1) {
    // this share's sums, not normalized, with the wave's own max and sum beside them
    const int64_t row = ((int64_t)split * num_tokens + t_first + my_tok) * heads + h0 + my_head;
    if (hf == 0) {
      part_ml[(row * 4 + w) * 2] = m;
      part_ml[(row * 4 + w) * 2 + 1] = l;
    }
#pragma unroll
    for (int n = 0; n < VBW; ++n) {
      const int blk = w + 4 * n;
      if (blk < vb) {
#pragma unroll
        for (int i = 0; i < 16; ++i) part_o[row * rank + 32 * blk + (i & 3) + 8 * (i >> 2) + 4 * hf] = o[n][i];
      }
    }
    return;
  }
  float inv = 1.f / l;
  if (gate != nullptr) inv /= 1.f + expf(-S::to_f32(gate[(int64_t)(t_first + my_tok) * gate_stride + h0 + my_head]));
  T* orow = out + (int64_t)(t_first + my_tok) * out_token_stride + (int64_t)(h0 + my_head) * out_head_stride;
#pragma unroll
  for (int n = 0; n < VBW; ++n) {
    const int blk = w + 4 * n;
    if (blk < vb) {
#pragma unroll
      for (int i = 0; i < 16; ++i)
        orow[32 * blk + (i & 3) + 8 * (i >> 2) + 4 * hf] = S::from_f32(o[n][i] * inv);
    }
  }
}

// out[t, h, d] = sum_s o_s[d] 2^(m_s - M) / sum_s l_s 2^(m_s - M) over the key shares s, M the
// largest m_s; the block of 32 dims d belongs to wave (d / 32) % 4 of the shares' workgroups
template <class S>
__global__ __launch_bounds__(256) void latent_merge_kernel(
    typename S::T* __restrict__ out, int64_t out_token_stride, int64_t out_head_stride,
    const float* __restrict__ part_o, const float* __restrict__ part_ml, int key_splits,
    int num_tokens, int heads, int rank, const typename S::T* __restrict__ gate, int64_t gate_stride) {
  const int64_t th = blockIdx.x;                 // token * heads + head
  const int64_t t = th / heads;
  const int h = (int)(th - t * heads);
  const float gv = gate != nullptr ? 1.f / (1.f + expf(-S::to_f32(gate[t * gate_stride + h]))) : 1.f;
  for (int d = threadIdx.x; d < rank; d += blockDim.x) {
    const int w = (d >> 5) & 3;
    const int64_t stride = (int64_t)num_tokens * heads;        // rows between two shares
    const float* ml = part_ml + ((t * heads + h) * 4 + w) * 2;
    const float* po = part_o + (t * heads + h) * rank + d;
    float big = -INFINITY;
#pragma unroll 8
    for (int sp = 0; sp < key_splits; ++sp) big = fmaxf(big, ml[sp * stride * 8]);
    float num = 0.f, den = 0.f;
#pragma unroll 8
    for (int sp = 0; sp < key_splits; ++sp) {
      const float ms = ml[sp * stride * 8], ls = ml[sp * stride * 8 + 1], ov = po[sp * stride * rank];
      const float f = ms == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ms - big);   // an empty share
      num += ov * f;
      den += ls * f;
    }
    out[t * out_token_stride + h * out_head_stride + d] = S::from_f32(num / den * gv);
  }
}

std::atomic<int> g_latent_kernel{0};

bool latent_tile_sizes(int rank, int rot) {
  if (rank % 32 != 0 || rank < 32 || rank > 512 || rot % 16 != 0) return false;
  const int vbw = (rank / 32 + 3) / 4;
  return (rank + rot) * kTileKeys / 8 <= 256 * (2 * vbw + 2);
}

template <class S, int VBW>
int launch_latent_tiles(dim3 grid, size_t lds, hipStream_t stream, typename S::T* out,
                        int64_t out_token_stride, int64_t out_head_stride, const LatentQuery<S>& q,
                        const typename S::T* cache, const int* block_tables, int max_blocks,
                        const int* qsl, const int* ctx, int heads, int rank, int rot, int block_size,
                        int num_blocks, float scale, int hb, int tb, int key_splits, float* part_o,
                        float* part_ml, int num_tokens, int window, const typename S::T* gate,
                        int64_t gate_stride) {
  static std::atomic<size_t> allowed{64 * 1024};   // raised once per kernel, not per launch
  if (lds > allowed.load(std::memory_order_relaxed)) {
    VLA_SEQ_HIP_CHECK(hipFuncSetAttribute(
        reinterpret_cast<const void*>(&latent_attention_tile_kernel<S, VBW>),
        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    allowed.store(lds, std::memory_order_relaxed);
  }
  latent_attention_tile_kernel<S, VBW><<<grid, 256, lds, stream>>>(
      out, out_token_stride, out_head_stride, q, cache, block_tables, max_blocks, qsl, ctx, heads,
      rank, rot, block_size, num_blocks, scale, hb, tb, key_splits, part_o, part_ml, num_tokens,
      window, gate, gate_stride);
  VLA_SEQ_HIP_CHECK(hipGetLastError());
  if (key_splits > 1) {
    latent_merge_kernel<S><<<(unsigned)((int64_t)num_tokens * heads), 256, 0, stream>>>(
        out, out_token_stride, out_head_stride, part_o, part_ml, key_splits, num_tokens, heads, rank,
        gate, gate_stride);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
  }
  return VLA_OK;
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
                                           int interleaved, void* stream) {
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
        (int64_t)num_blocks * block_size, interleaved);
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
                                        int num_blocks, float scale, int dtype, int window,
                                        const void* gate, int64_t gate_stride, void* stream) {
  if (num_tokens == 0) return VLA_OK;
  if (gate && gate_stride < heads) return VLA_ERR_ARG;
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
        token_seq, positions, heads, rank, rot, block_size, num_blocks, scale, window, (const T*)gate,
        gate_stride);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}

// 0: pick per shape; 1: never the matrix-core kernel (tests run both)
extern "C" int vla_seq_set_latent_attention_kernel(int mode) {
  if (mode < 0 || mode > 1) return VLA_ERR_ARG;
  g_latent_kernel.store(mode, std::memory_order_relaxed);
  return VLA_OK;
}

extern "C" int vla_seq_latent_attention_tiles_supported(int rank, int rot, int dtype) {
  return (dtype == VLA_F16 || dtype == VLA_BF16) && latent_tile_sizes(rank, rot) &&
         g_latent_kernel.load(std::memory_order_relaxed) == 0;
}

extern "C" int64_t vla_seq_latent_attention_scratch_floats(int key_splits, int num_tokens, int heads,
                                                           int rank) {
  return key_splits > 1 ? (int64_t)key_splits * num_tokens * heads * (rank + 8) : 0;
}

extern "C" int vla_seq_latent_attention_tiles(
    void* out, int64_t out_token_stride, int64_t out_head_stride, const void* q_lat,
    int64_t lat_token_stride, int64_t lat_head_stride, const void* q_rot, int64_t rot_token_stride,
    int64_t rot_head_stride, const void* cache, const int* block_tables, int max_blocks,
    const int* query_start_loc, const int* context_lens, int num_seqs, int max_query_len, int heads,
    int rank, int rot, int block_size, int num_blocks, float scale, int key_splits, float* scratch,
    int num_tokens, int dtype, int window, const void* gate, int64_t gate_stride, void* stream) {
  if (num_seqs == 0 || max_query_len == 0) return VLA_OK;
  if (gate && gate_stride < heads) return VLA_ERR_ARG;
  if (!out || !q_lat || (rot > 0 && !q_rot) || !cache || !block_tables || !query_start_loc ||
      !context_lens || num_seqs < 0 || num_seqs > 65535 || max_query_len < 0 || heads <= 0 ||
      rot < 0 || block_size <= 0 || num_blocks <= 0 || max_blocks <= 0 || key_splits < 1 ||
      key_splits > 64 || (key_splits > 1 && (!scratch || num_tokens <= 0)))
    return VLA_ERR_ARG;
  if ((dtype != VLA_F16 && dtype != VLA_BF16) || !latent_tile_sizes(rank, rot)) return VLA_ERR_HEAD_SIZE;
  // 16-byte fragment loads: query rows and cache rows must allow them
  if (((uintptr_t)q_lat % 16) || (lat_token_stride % 8) || (lat_head_stride % 8) || ((uintptr_t)cache % 16) ||
      (rot > 0 && (((uintptr_t)q_rot % 16) || (rot_token_stride % 8) || (rot_head_stride % 8))))
    return VLA_ERR_ARG;
  const int hb = heads < kTileRows ? heads : kTileRows;     // heads of a workgroup's rows
  const int tb = kTileRows / hb;                            // tokens of a workgroup's rows
  const dim3 grid((max_query_len + tb - 1) / tb * key_splits, (heads + hb - 1) / hb, num_seqs);
  // scratch: the shares' sums [key_splits, T, heads, rank], then their max / sum per wave
  float* part_o = scratch;
  float* part_ml = scratch ? scratch + (int64_t)key_splits * num_tokens * heads * rank : nullptr;
  const int row_elems = rank + rot + 8;
  const size_t lds = (size_t)kTileKeys * row_elems * 2 + 4 * 16 * 64 * sizeof(float) +
                     2 * kTileKeys * sizeof(long long);
  if (lds > 160 * 1024) return VLA_ERR_HEAD_SIZE;
  const int vbw = (rank / 32 + 3) / 4;
  auto go = [&](auto s) {
    using S = decltype(s);
    using T = typename S::T;
    const LatentQuery<S> q{(const T*)q_lat, lat_token_stride, lat_head_stride, (const T*)q_rot,
                           rot_token_stride, rot_head_stride};
#define VLA_LATENT_CASE(N)                                                                          \
  case N:                                                                                           \
    return launch_latent_tiles<S, N>(grid, lds, (hipStream_t)stream, (T*)out, out_token_stride,     \
                                     out_head_stride, q, (const T*)cache, block_tables, max_blocks, \
                                     query_start_loc, context_lens, heads, rank, rot, block_size,   \
                                     num_blocks, scale, hb, tb, key_splits, part_o, part_ml,        \
                                     num_tokens, window, (const T*)gate, gate_stride);
    switch (vbw) {
      VLA_LATENT_CASE(1)
      VLA_LATENT_CASE(2)
      VLA_LATENT_CASE(3)
      VLA_LATENT_CASE(4)
      default: return (int)VLA_ERR_HEAD_SIZE;
    }
#undef VLA_LATENT_CASE
  };
  return dtype == VLA_BF16 ? go(BF16{}) : go(F16{});
}
