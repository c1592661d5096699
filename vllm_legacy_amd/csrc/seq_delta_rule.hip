// Gated delta rule: per head a state S [dim, vdim] in fp32 that every token first decays, then
// corrects towards its value along its key, then reads with its query:
//   S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
// with k and q made unit vectors per head (q also times dim^-1/2), beta = sigmoid(b),
// g = exp(-exp(A_log) softplus(dt + dt_bias)).  The head's o is RMS-normed over vdim, weighted and
// gated with silu before it leaves.  Several value heads may share one query / key head.
//
// One workgroup per (head, sequence, group of value columns) walks the sequence's rows of the step.
// A column of S (one value dimension) never meets another, so a head's columns are spread over
// workgroups, and thread (j, r) keeps R rows of column j in registers -- rows 4 (ii split + r) ..
// + 3 for ii < R / 4, so that the `split` threads of a column, neighbours in a wave, read whole
// lines of the state and of the staged keys -- and they add their partial dot products with lane
// exchanges.  Rows go through LDS in chunks: queries, keys, values and the per-token numbers of a
// chunk are staged and normed together, and the walk then needs no barrier per token.  With
//   dk = S^T k and dq = S^T q taken from the state before the token,
//   u = beta (v - g dk),   o = g dq + (k . q) u,   S <- g S + k u^T
// is the same update with both dot products read from one state.  Steps whose runs have at most
// four rows (decode steps) skip the staging: the lanes of a column read their rows of the query and
// key themselves and the unit norms are lane sums.  The walk leaves o in fp32; a
// second launch norms each head's o over vdim, weighs and gates it.  The state is stored
// [slot, head, vdim, dim], so a thread's rows are contiguous.  Everything is fp32.
#include <algorithm>
#include <atomic>

#include "seq_common.h"

namespace vla {
namespace seq {
namespace {

constexpr int kMaxChunk = 32;
constexpr int kMaxSplit = 16;

// v + the value another lane holds, the lanes paired by a DPP pattern (no LDS round trip)
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
  const int other = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false);
  return v + __builtin_bit_cast(float, other);
}

// the sum over each aligned group of `split` lanes (1, 2, 4, 8 or 16), in every lane of the group:
// neighbours, pairs of a quad, the mirrored half of eight, the mirrored half of sixteen
__device__ __forceinline__ void group_sums(float& a, float& b, int split) {
  if (split > 1) {
    a = dpp_add<0xB1>(a);      // quad_perm [1, 0, 3, 2]
    b = dpp_add<0xB1>(b);
  }
  if (split > 2) {
    a = dpp_add<0x4E>(a);      // quad_perm [2, 3, 0, 1]
    b = dpp_add<0x4E>(b);
  }
  if (split > 4) {
    a = dpp_add<0x141>(a);     // row_half_mirror: lane i of eight with lane 7 - i
    b = dpp_add<0x141>(b);
  }
  if (split > 8) {
    a = dpp_add<0x140>(a);     // row_mirror: lane i of sixteen with lane 15 - i
    b = dpp_add<0x140>(b);
  }
}

__device__ __forceinline__ float softplusf(float z) { return z > 20.f ? z : log1pf(expf(z)); }

template <class SI>
struct DeltaRows {
  const typename SI::T* q;
  int64_t q_stride;
  const typename SI::T* k;
  int64_t k_stride;
  const typename SI::T* v;
  int64_t v_stride;
  const typename SI::T* gate;
  int64_t gate_stride;
  const typename SI::T* beta;
  int64_t beta_stride;
  const typename SI::T* dt;
  int64_t dt_stride;
};

template <class SI, int R>
__global__ __launch_bounds__(256) void delta_rule_kernel(
    float* __restrict__ o, DeltaRows<SI> in, const float* __restrict__ a_log,
    const float* __restrict__ dt_bias, float* __restrict__ state,
    const int* __restrict__ query_start_loc, const int* __restrict__ context_lens,
    const int* __restrict__ state_slots, int heads, int kv_heads, int dim, int vdim, int split,
    int cols, int chunk) {
  extern __shared__ __align__(16) float lds[];
  const int dp = split * R;                       // padded dim
  float* q_lds = lds;                             // [chunk][dp]
  float* k_lds = q_lds + chunk * dp;              // [chunk][dp]
  float* v_lds = k_lds + chunk * dp;              // [chunk][cols]
  float* num = v_lds + chunk * cols;              // [chunk][5]: g, beta, k scale, q scale, k . q

  // the column group runs fastest: workgroups that run together touch one stretch of the state
  const int h = blockIdx.y, b = blockIdx.z, j0 = blockIdx.x * cols;
  const int g_head = h / (heads / kv_heads);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, waves = blockDim.x >> 6;
  const int jl = tid / split, r = tid - jl * split;
  const int j = j0 + jl;
  const bool col = jl < cols && j < vdim;
  const int ncols = min(cols, vdim - j0);
  const int start = query_start_loc[b], end = query_start_loc[b + 1];
  float* st = state + (((int64_t)state_slots[b] * heads + h) * vdim + (col ? j : 0)) * dim;
  const bool whole = dim == dp && (dim & 3) == 0;  // no padded rows: four rows per access
  const bool resume = context_lens[b] > 0;
  float s[R];
#pragma unroll
  for (int ii = 0; ii < R / 4; ++ii) {
    const int d = 4 * (ii * split + r);
    f32x4 got = {0.f, 0.f, 0.f, 0.f};
    if (col && resume) {
      if (whole) {
        got = *reinterpret_cast<const f32x4*>(st + d);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (d + e < dim) got[e] = st[d + e];
      }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) s[4 * ii + e] = got[e];
  }
  const float decay_rate = expf(a_log[h]), bias = dt_bias[h];
  const float q_unit = 1.f / sqrtf((float)dim);

  // A chunk's rows come through registers: they are asked for before the walk over the chunk
  // ahead of them, and land in LDS when that walk is done.
  constexpr int PF = 8;                           // pieces of four rows / of values a thread stages
  f32x4 pq[PF], pk[PF];
  float pv[PF], pb = 0.f, pd = 0.f;
  const int quads = dp / 4;                        // a power of two, as split and R are
  const int quad_shift = __ffs(quads) - 1;
  const bool vec = whole && (in.q_stride & 3) == 0 && (in.k_stride & 3) == 0 &&
                   ((uintptr_t)in.q & 15) == 0 && ((uintptr_t)in.k & 15) == 0;
  auto fetch = [&](int t0, int n) {
    const int pieces = max(n * quads, n * ncols);
#pragma unroll
    for (int u = 0; u < PF; ++u) {
      if (u * (int)blockDim.x >= pieces) break;    // a short chunk (a decode step) stops early
      const int i = tid + u * blockDim.x;
      f32x4 q4 = {0.f, 0.f, 0.f, 0.f}, k4 = {0.f, 0.f, 0.f, 0.f};
      if (i < n * quads) {
        const int tc = i >> quad_shift, d = 4 * (i & (quads - 1));
        const typename SI::T* qr = in.q + (int64_t)(t0 + tc) * in.q_stride + (int64_t)g_head * dim + d;
        const typename SI::T* kr = in.k + (int64_t)(t0 + tc) * in.k_stride + (int64_t)g_head * dim + d;
        if (vec) {
          q4 = *reinterpret_cast<const f32x4*>(qr);
          k4 = *reinterpret_cast<const f32x4*>(kr);
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (d + e < dim) {
              q4[e] = SI::to_f32(qr[e]);
              k4[e] = SI::to_f32(kr[e]);
            }
        }
      }
      pq[u] = q4;
      pk[u] = k4;
      pv[u] = 0.f;
      if (i < n * ncols) {
        const int tc = i / ncols, d = i - tc * ncols;
        pv[u] = SI::to_f32(in.v[(int64_t)(t0 + tc) * in.v_stride + (int64_t)h * vdim + j0 + d]);
      }
    }
    if (tid < n) {
      pb = SI::to_f32(in.beta[(int64_t)(t0 + tid) * in.beta_stride + h]);
      pd = SI::to_f32(in.dt[(int64_t)(t0 + tid) * in.dt_stride + h]);
    }
  };
  auto land = [&](int n) {
    const int pieces = max(n * quads, n * ncols);
#pragma unroll
    for (int u = 0; u < PF; ++u) {
      if (u * (int)blockDim.x >= pieces) break;
      const int i = tid + u * blockDim.x;
      if (i < n * quads) {
        *reinterpret_cast<f32x4*>(q_lds + 4 * i) = pq[u];
        *reinterpret_cast<f32x4*>(k_lds + 4 * i) = pk[u];
      }
      if (i < n * ncols) {
        const int tc = i / ncols, d = i - tc * ncols;
        v_lds[tc * cols + d] = pv[u];
      }
    }
    if (tid < n) {
      num[tid * 5 + 0] = expf(-decay_rate * softplusf(pd + bias));
      num[tid * 5 + 1] = 1.f / (1.f + expf(-pb));
    }
  };
  // the unit norms of a chunk's queries and keys and their product: four lanes per token, each
  // summing every fourth row (a token's walk starts 4 tc rows in, so that the tokens of a wave
  // read different banks; the padded rows are zeros)
  auto norms = [&](int n) {
    const int tc = tid >> 2, part = tid & 3;
    float qq = 0.f, kk = 0.f, kq = 0.f;
    if (tc < n) {
      int d = (part + 4 * tc) & (dp - 1);
#pragma unroll 8
      for (int i = 0; i < quads; ++i) {
        const float qv = q_lds[tc * dp + d], kv = k_lds[tc * dp + d];
        qq += qv * qv;
        kk += kv * kv;
        kq += kv * qv;
        d += 4;
        d = d >= dp ? d - dp : d;
      }
    }
    qq = dpp_add<0x4E>(dpp_add<0xB1>(qq));
    kk = dpp_add<0x4E>(dpp_add<0xB1>(kk));
    kq = dpp_add<0x4E>(dpp_add<0xB1>(kq));
    if (tc < n && part == 0) {
      const float ks = 1.f / sqrtf(kk + 1e-6f), qs = q_unit / sqrtf(qq + 1e-6f);
      num[tc * 5 + 2] = ks;
      num[tc * 5 + 3] = qs;
      num[tc * 5 + 4] = kq * ks * qs;
    }
  };
  fetch(start, min(chunk, end - start));
  land(min(chunk, end - start));
  __syncthreads();
  norms(min(chunk, end - start));
  __syncthreads();
  for (int t0 = start; t0 < end; t0 += chunk) {
    const int n = min(chunk, end - t0);
    const int n_next = min(chunk, end - t0 - chunk);
    if (n_next > 0) fetch(t0 + chunk, n_next);
    float* orow = o + ((int64_t)t0 * heads + h) * vdim + (col ? j : 0);
    for (int tc = 0; tc < n; ++tc) {
      const float g = num[tc * 5 + 0], be = num[tc * 5 + 1], ks = num[tc * 5 + 2], qs = num[tc * 5 + 3],
                  kq = num[tc * 5 + 4];
      float kv[R];
      float dk0 = 0.f, dk1 = 0.f, dq0 = 0.f, dq1 = 0.f;
#pragma unroll
      for (int ii = 0; ii < R / 4; ++ii) {
        const f32x4 k4 = *reinterpret_cast<const f32x4*>(k_lds + tc * dp + 4 * (ii * split + r));
        const f32x4 q4 = *reinterpret_cast<const f32x4*>(q_lds + tc * dp + 4 * (ii * split + r));
#pragma unroll
        for (int e = 0; e < 4; e += 2) {
          kv[4 * ii + e] = k4[e];
          kv[4 * ii + e + 1] = k4[e + 1];
          dk0 += s[4 * ii + e] * k4[e];
          dk1 += s[4 * ii + e + 1] * k4[e + 1];
          dq0 += s[4 * ii + e] * q4[e];
          dq1 += s[4 * ii + e + 1] * q4[e + 1];
        }
      }
      float dk = dk0 + dk1, dq = dq0 + dq1;
      group_sums(dk, dq, split);
      const float u = be * (v_lds[tc * cols + (col ? jl : 0)] - g * ks * dk);
      const float ku = ks * u;
#pragma unroll
      for (int i = 0; i < R; ++i) s[i] = g * s[i] + kv[i] * ku;
      if (col && r == 0) orow[(int64_t)tc * heads * vdim] = g * qs * dq + kq * u;
    }
    if (n_next > 0) {
      __syncthreads();
      land(n_next);
      __syncthreads();
      norms(n_next);
      __syncthreads();
    }
  }
  if (col) {
#pragma unroll
    for (int ii = 0; ii < R / 4; ++ii) {
      const int d = 4 * (ii * split + r);
      if (whole) {
        const f32x4 put = {s[4 * ii], s[4 * ii + 1], s[4 * ii + 2], s[4 * ii + 3]};
        *reinterpret_cast<f32x4*>(st + d) = put;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (d + e < dim) st[d + e] = s[4 * ii + e];
      }
    }
  }
}

// Runs of a few rows (decode steps): no staging.  The `split` lanes of a column hold all rows between
// them, so a token's unit norms are lane sums of what they read for the dot products anyway.
template <class SI, int R>
__global__ __launch_bounds__(256) void delta_rule_step_kernel(
    float* __restrict__ o, DeltaRows<SI> in, const float* __restrict__ a_log,
    const float* __restrict__ dt_bias, float* __restrict__ state,
    const int* __restrict__ query_start_loc, const int* __restrict__ context_lens,
    const int* __restrict__ state_slots, int heads, int kv_heads, int dim, int vdim, int split,
    int cols) {
  const int h = blockIdx.y, b = blockIdx.z, j0 = blockIdx.x * cols;
  const int g_head = h / (heads / kv_heads);
  const int tid = threadIdx.x;
  const int jl = tid / split, r = tid - jl * split;
  const int j = j0 + jl;
  const bool col = jl < cols && j < vdim;
  const int start = query_start_loc[b], end = query_start_loc[b + 1];
  float* st = state + (((int64_t)state_slots[b] * heads + h) * vdim + (col ? j : 0)) * dim;
  const bool whole = dim == split * R && (dim & 3) == 0;
  const bool vec = whole && (in.q_stride & 3) == 0 && (in.k_stride & 3) == 0 &&
                   ((uintptr_t)in.q & 15) == 0 && ((uintptr_t)in.k & 15) == 0;
  const bool resume = context_lens[b] > 0;
  float s[R];
#pragma unroll
  for (int ii = 0; ii < R / 4; ++ii) {
    const int d = 4 * (ii * split + r);
    f32x4 got = {0.f, 0.f, 0.f, 0.f};
    if (col && resume) {
      if (whole) {
        got = *reinterpret_cast<const f32x4*>(st + d);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (d + e < dim) got[e] = st[d + e];
      }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) s[4 * ii + e] = got[e];
  }
  const float decay_rate = expf(a_log[h]), bias = dt_bias[h];
  const float q_unit = 1.f / sqrtf((float)dim);
  for (int t = start; t < end; ++t) {
    float kv[R], qv[R];
#pragma unroll
    for (int ii = 0; ii < R / 4; ++ii) {
      const int d = 4 * (ii * split + r);
      const typename SI::T* qr = in.q + (int64_t)t * in.q_stride + (int64_t)g_head * dim + d;
      const typename SI::T* kr = in.k + (int64_t)t * in.k_stride + (int64_t)g_head * dim + d;
      f32x4 q4 = {0.f, 0.f, 0.f, 0.f}, k4 = {0.f, 0.f, 0.f, 0.f};
      if (vec) {
        q4 = *reinterpret_cast<const f32x4*>(qr);
        k4 = *reinterpret_cast<const f32x4*>(kr);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (d + e < dim) {
            q4[e] = SI::to_f32(qr[e]);
            k4[e] = SI::to_f32(kr[e]);
          }
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        qv[4 * ii + e] = q4[e];
        kv[4 * ii + e] = k4[e];
      }
    }
    const float vj = SI::to_f32(in.v[(int64_t)t * in.v_stride + (int64_t)h * vdim + (col ? j : 0)]);
    const float be = 1.f / (1.f + expf(-SI::to_f32(in.beta[(int64_t)t * in.beta_stride + h])));
    const float g = expf(-decay_rate * softplusf(SI::to_f32(in.dt[(int64_t)t * in.dt_stride + h]) + bias));
    float qq = 0.f, kk = 0.f, kq = 0.f, dk = 0.f, dq = 0.f, none = 0.f;
#pragma unroll
    for (int i = 0; i < R; ++i) {
      qq += qv[i] * qv[i];
      kk += kv[i] * kv[i];
      kq += kv[i] * qv[i];
      dk += s[i] * kv[i];
      dq += s[i] * qv[i];
    }
    group_sums(qq, kk, split);
    group_sums(kq, none, split);
    group_sums(dk, dq, split);
    const float ks = 1.f / sqrtf(kk + 1e-6f), qs = q_unit / sqrtf(qq + 1e-6f);
    const float u = be * (vj - g * ks * dk);
    const float ku = ks * u;
#pragma unroll
    for (int i = 0; i < R; ++i) s[i] = g * s[i] + kv[i] * ku;
    if (col && r == 0) o[((int64_t)t * heads + h) * vdim + j] = g * qs * dq + kq * ks * qs * u;
  }
  if (col) {
#pragma unroll
    for (int ii = 0; ii < R / 4; ++ii) {
      const int d = 4 * (ii * split + r);
      if (whole) {
        const f32x4 put = {s[4 * ii], s[4 * ii + 1], s[4 * ii + 2], s[4 * ii + 3]};
        *reinterpret_cast<f32x4*>(st + d) = put;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (d + e < dim) st[d + e] = s[4 * ii + e];
      }
    }
  }
}

// out = dtype(o / sqrt(mean_v(o^2) + eps) * weight * silu(gate)) per (token, head): one wave each
template <class SI, class SO>
__global__ __launch_bounds__(256) void delta_head_norm_kernel(
    typename SO::T* __restrict__ out, int64_t out_stride, const float* __restrict__ o,
    const typename SI::T* __restrict__ gate, int64_t gate_stride, const float* __restrict__ weight,
    float eps, int rows, int heads, int vdim) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);     // token * heads + head
  if (row >= rows) return;
  const int64_t t = row / heads;
  const int h = (int)(row - t * heads);
  const float* orow = o + row * vdim;
  float ss = 0.f;
  for (int d = lane; d < vdim; d += kWave) ss += orow[d] * orow[d];
  ss = wave_sum(ss);
  const float inv = 1.f / sqrtf(ss / (float)vdim + eps);
  for (int d = lane; d < vdim; d += kWave) {
    const float gt = SI::to_f32(gate[t * gate_stride + (int64_t)h * vdim + d]);
    out[t * out_stride + (int64_t)h * vdim + d] = SO::from_f32(orow[d] * inv * weight[d] * (gt / (1.f + expf(-gt))));
  }
}

std::atomic<int> g_delta_kernel{0};

int pow2_at_least(int n) {
  int p = 1;
  while (p < n) p <<= 1;
  return p;
}

}  // namespace
}  // namespace seq
}  // namespace vla

using namespace vla;
using namespace vla::seq;

extern "C" int64_t vla_seq_delta_rule_scratch_floats(int num_tokens, int heads, int vdim) {
  return (int64_t)num_tokens * heads * vdim;
}

extern "C" int vla_seq_delta_rule_scan(
    void* out, int64_t out_stride, int out_dtype, const void* q, int64_t q_stride, const void* k,
    int64_t k_stride, const void* v, int64_t v_stride, const void* gate, int64_t gate_stride,
    const void* beta, int64_t beta_stride, const void* dt, int64_t dt_stride, int in_dtype,
    const float* a_log, const float* dt_bias, const float* norm_weight, float* state,
    const int* query_start_loc, const int* context_lens, const int* state_slots, int num_tokens,
    int num_seqs, int max_query_len, int num_slots, int heads, int kv_heads, int dim, int vdim,
    float eps, float* scratch, void* stream) {
  if (num_seqs == 0 || num_tokens == 0) return VLA_OK;
  if (!out || !q || !k || !v || !gate || !beta || !dt || !a_log || !dt_bias || !norm_weight ||
      !state || !scratch || !query_start_loc || !context_lens || !state_slots || num_seqs < 0 ||
      num_seqs > 65535 || num_tokens < 0 || num_slots <= 0 || heads <= 0 || kv_heads <= 0 ||
      heads % kv_heads != 0 || dim <= 0 || vdim <= 0 || out_stride < (int64_t)heads * vdim ||
      q_stride < (int64_t)kv_heads * dim || k_stride < (int64_t)kv_heads * dim ||
      v_stride < (int64_t)heads * vdim || gate_stride < (int64_t)heads * vdim ||
      beta_stride < heads || dt_stride < heads)
    return VLA_ERR_ARG;
  // the rows that enter the recurrence are fp32 (the caller's projections leave them so)
  if (in_dtype != VLA_F32) return VLA_ERR_DTYPE;
  // the fewest rows per thread (8, 16, 32, 64) whose column groups are at most kMaxSplit lanes
  int rows = 0, split = 0;
  for (int r = 8; r <= 64; r *= 2) {
    const int sp = pow2_at_least((dim + r - 1) / r);
    if (sp <= kMaxSplit) {
      rows = r;
      split = sp;
      break;
    }
  }
  if (rows == 0) return VLA_ERR_HEAD_SIZE;
  // a workgroup of 256 threads: 256 / split columns of one head
  const int cols = 256 / split < vdim ? 256 / split : vdim;
  const int threads = (cols * split + 63) / 64 * 64;
  const int col_groups = (vdim + cols - 1) / cols;
  if (heads > 65535) return VLA_ERR_ARG;
  // a chunk fits LDS, a thread's staging registers (8 pieces of four rows, 8 values) and four
  // threads per token
  const size_t per_token = (size_t)(2 * split * rows + cols + 5) * sizeof(float);
  int chunk = kMaxChunk;
  chunk = std::min<int64_t>(chunk, 60 * 1024 / per_token);
  chunk = std::min(chunk, 8 * threads * 4 / (split * rows));
  chunk = std::min(chunk, 8 * threads / cols);
  chunk = std::min(chunk, threads / 4);
  if (max_query_len > 0) chunk = std::min(chunk, max_query_len);
  if (chunk < 1) return VLA_ERR_HEAD_SIZE;
  const size_t lds = chunk * per_token;
  using SI = F32;
  const DeltaRows<SI> in{(const float*)q, q_stride, (const float*)k, k_stride, (const float*)v, v_stride,
                         (const float*)gate, gate_stride, (const float*)beta, beta_stride,
                         (const float*)dt, dt_stride};
  const dim3 grid(col_groups, heads, num_seqs);
  // runs of at most four rows take the kernel without staging (modes 1 / 2: always / never, for tests)
  const int mode = g_delta_kernel.load(std::memory_order_relaxed);
  const bool steps = mode == 1 || (mode == 0 && max_query_len > 0 && max_query_len <= 4);
  if (steps) {
    auto launch_step = [&](auto kernel) {
      kernel<<<grid, threads, 0, (hipStream_t)stream>>>(scratch, in, a_log, dt_bias, state, query_start_loc,
                                                        context_lens, state_slots, heads, kv_heads, dim, vdim,
                                                        split, cols);
    };
    switch (rows) {
      case 8: launch_step(delta_rule_step_kernel<SI, 8>); break;
      case 16: launch_step(delta_rule_step_kernel<SI, 16>); break;
      case 32: launch_step(delta_rule_step_kernel<SI, 32>); break;
      default: launch_step(delta_rule_step_kernel<SI, 64>); break;
    }
  }
  auto launch = [&](auto kernel) {
    kernel<<<grid, threads, lds, (hipStream_t)stream>>>(scratch, in, a_log, dt_bias, state, query_start_loc,
                                                        context_lens, state_slots, heads, kv_heads, dim,
                                                        vdim, split, cols, chunk);
  };
  if (!steps) {
    switch (rows) {
      case 8: launch(delta_rule_kernel<SI, 8>); break;
      case 16: launch(delta_rule_kernel<SI, 16>); break;
      case 32: launch(delta_rule_kernel<SI, 32>); break;
      default: launch(delta_rule_kernel<SI, 64>); break;
    }
  }
  VLA_SEQ_HIP_CHECK(hipGetLastError());
  return with_dtype(out_dtype, [&](auto so) {
    using SO = decltype(so);
    const int64_t head_rows = (int64_t)num_tokens * heads;
    delta_head_norm_kernel<SI, SO><<<(unsigned)((head_rows + 3) / 4), 256, 0, (hipStream_t)stream>>>(
        (typename SO::T*)out, out_stride, scratch, (const float*)gate, gate_stride, norm_weight, eps,
        (int)head_rows, heads, vdim);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}

// 0: pick per step; 1: always the kernel without staging; 2: never (tests run both)
extern "C" int vla_seq_set_delta_kernel(int mode) {
  if (mode < 0 || mode > 2) return VLA_ERR_ARG;
  g_delta_kernel.store(mode, std::memory_order_relaxed);
  return VLA_OK;
}
