// Gated delta rule: per head a state S [dim, vdim] in fp32 that every token first decays, then
// corrects towards its value along its key, then reads with its query:
//   S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
// with k and q made unit vectors per head (q also times dim^-1/2), beta = sigmoid(b),
// g = exp(-exp(A_log) softplus(dt + dt_bias)).  The head's o is RMS-normed over vdim, weighted and
// gated with silu before it leaves.  Several value heads may share one query / key head.
//
// One workgroup per (head, sequence) walks the sequence's rows of the step.  A column of S (one
// value dimension) never meets another, so thread (j, r) keeps rows r R .. r R + R - 1 of column
// j in registers; the `split` threads of a column are neighbours in a wave and add their partial
// dot products with lane exchanges.  Rows go through LDS in chunks: queries, keys, values and the
// per-token numbers of a chunk are staged and normed together, the walk then needs no barrier
// per token, and the chunk's outputs are normed, gated and written together.  With
//   dk = S^T k and dq = S^T q taken from the state before the token,
//   u = beta (v - g dk),   o = g dq + (k . q) u,   S <- g S + k u^T
// is the same update with both dot products read from one state.  The state is stored
// [slot, head, vdim, dim], so a thread's rows are contiguous.  Everything is fp32.
#include "seq_common.h"

namespace vla {
namespace seq {
namespace {

constexpr int kChunk = 16;

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

template <class SI, class SO, int R>
__global__ __launch_bounds__(1024) void delta_rule_kernel(
    typename SO::T* __restrict__ out, int64_t out_stride, DeltaRows<SI> in,
    const float* __restrict__ a_log, const float* __restrict__ dt_bias,
    const float* __restrict__ norm_weight, float* __restrict__ state,
    const int* __restrict__ query_start_loc, const int* __restrict__ context_lens,
    const int* __restrict__ state_slots, int heads, int kv_heads, int dim, int vdim, int split,
    float eps) {
  extern __shared__ __align__(16) float lds[];
  const int dp = split * R;                       // padded dim
  float* q_lds = lds;                             // [kChunk][dp]
  float* k_lds = q_lds + kChunk * dp;             // [kChunk][dp]
  float* v_lds = k_lds + kChunk * dp;             // [kChunk][vdim]
  float* o_lds = v_lds + kChunk * vdim;           // [kChunk][vdim]
  float* num = o_lds + kChunk * vdim;             // [kChunk][5]: g, beta, k scale, q scale, k . q

  const int h = blockIdx.x, b = blockIdx.y;
  const int g_head = h / (heads / kv_heads);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, waves = blockDim.x >> 6;
  const int j = tid / split, r = tid - j * split;
  const bool col = j < vdim;
  const int start = query_start_loc[b], end = query_start_loc[b + 1];
  float* st = state + (((int64_t)state_slots[b] * heads + h) * vdim + (col ? j : 0)) * dim;
  float s[R];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int d = r * R + i;
    s[i] = col && d < dim && context_lens[b] > 0 ? st[d] : 0.f;
  }
  const float decay_rate = expf(a_log[h]), bias = dt_bias[h];
  const float q_unit = 1.f / sqrtf((float)dim);

  for (int t0 = start; t0 < end; t0 += kChunk) {
    const int n = min(kChunk, end - t0);
    for (int i = tid; i < n * dp; i += blockDim.x) {
      const int tc = i / dp, d = i - tc * dp;
      float qv = 0.f, kv = 0.f;
      if (d < dim) {
        qv = SI::to_f32(in.q[(int64_t)(t0 + tc) * in.q_stride + (int64_t)g_head * dim + d]);
        kv = SI::to_f32(in.k[(int64_t)(t0 + tc) * in.k_stride + (int64_t)g_head * dim + d]);
      }
      q_lds[i] = qv;
      k_lds[i] = kv;
    }
    for (int i = tid; i < n * vdim; i += blockDim.x) {
      const int tc = i / vdim, d = i - tc * vdim;
      v_lds[i] = SI::to_f32(in.v[(int64_t)(t0 + tc) * in.v_stride + (int64_t)h * vdim + d]);
    }
    __syncthreads();
    for (int tc = wave; tc < n; tc += waves) {
      float qq = 0.f, kk = 0.f, kq = 0.f;
      for (int d = lane; d < dim; d += kWave) {
        const float qv = q_lds[tc * dp + d], kv = k_lds[tc * dp + d];
        qq += qv * qv;
        kk += kv * kv;
        kq += kv * qv;
      }
      qq = wave_sum(qq);
      kk = wave_sum(kk);
      kq = wave_sum(kq);
      if (lane == 0) {
        const float bp = SI::to_f32(in.beta[(int64_t)(t0 + tc) * in.beta_stride + h]);
        const float dtv = SI::to_f32(in.dt[(int64_t)(t0 + tc) * in.dt_stride + h]);
        const float ks = 1.f / sqrtf(kk + 1e-6f), qs = q_unit / sqrtf(qq + 1e-6f);
        num[tc * 5 + 0] = expf(-decay_rate * softplusf(dtv + bias));
        num[tc * 5 + 1] = 1.f / (1.f + expf(-bp));
        num[tc * 5 + 2] = ks;
        num[tc * 5 + 3] = qs;
        num[tc * 5 + 4] = kq * ks * qs;
      }
    }
    __syncthreads();
    for (int tc = 0; tc < n; ++tc) {
      const float g = num[tc * 5 + 0], be = num[tc * 5 + 1], ks = num[tc * 5 + 2], qs = num[tc * 5 + 3],
                  kq = num[tc * 5 + 4];
      const float* kr = k_lds + tc * dp + r * R;
      const float* qr = q_lds + tc * dp + r * R;
      float kv[R];
      float dk0 = 0.f, dk1 = 0.f, dq0 = 0.f, dq1 = 0.f;
#pragma unroll
      for (int i = 0; i < R; i += 2) {
        kv[i] = kr[i];
        kv[i + 1] = kr[i + 1];
        dk0 += s[i] * kv[i];
        dk1 += s[i + 1] * kv[i + 1];
        dq0 += s[i] * qr[i];
        dq1 += s[i + 1] * qr[i + 1];
      }
      float dk = dk0 + dk1, dq = dq0 + dq1;
      for (int m = 1; m < split; m <<= 1) {
        dk += __shfl_xor(dk, m, 64);
        dq += __shfl_xor(dq, m, 64);
      }
      const float u = be * (v_lds[tc * vdim + (col ? j : 0)] - g * ks * dk);
      const float ku = ks * u;
#pragma unroll
      for (int i = 0; i < R; ++i) s[i] = g * s[i] + kv[i] * ku;
      if (col && r == 0) o_lds[tc * vdim + j] = g * qs * dq + kq * u;
    }
    __syncthreads();
    for (int tc = wave; tc < n; tc += waves) {
      float ss = 0.f;
      for (int d = lane; d < vdim; d += kWave) ss += o_lds[tc * vdim + d] * o_lds[tc * vdim + d];
      ss = wave_sum(ss);
      const float inv = 1.f / sqrtf(ss / (float)vdim + eps);
      for (int d = lane; d < vdim; d += kWave) {
        const float gt = SI::to_f32(in.gate[(int64_t)(t0 + tc) * in.gate_stride + (int64_t)h * vdim + d]);
        out[(int64_t)(t0 + tc) * out_stride + (int64_t)h * vdim + d] =
            SO::from_f32(o_lds[tc * vdim + d] * inv * norm_weight[d] * (gt / (1.f + expf(-gt))));
      }
    }
    __syncthreads();
  }
  if (col) {
#pragma unroll
    for (int i = 0; i < R; ++i) {
      const int d = r * R + i;
      if (d < dim) st[d] = s[i];
    }
  }
}

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

extern "C" int vla_seq_delta_rule_scan(
    void* out, int64_t out_stride, int out_dtype, const void* q, int64_t q_stride, const void* k,
    int64_t k_stride, const void* v, int64_t v_stride, const void* gate, int64_t gate_stride,
    const void* beta, int64_t beta_stride, const void* dt, int64_t dt_stride, int in_dtype,
    const float* a_log, const float* dt_bias, const float* norm_weight, float* state,
    const int* query_start_loc, const int* context_lens, const int* state_slots, int num_seqs,
    int num_slots, int heads, int kv_heads, int dim, int vdim, float eps, void* stream) {
  if (num_seqs == 0) return VLA_OK;
  if (!out || !q || !k || !v || !gate || !beta || !dt || !a_log || !dt_bias || !norm_weight ||
      !state || !query_start_loc || !context_lens || !state_slots || num_seqs < 0 ||
      num_seqs > 65535 || num_slots <= 0 || heads <= 0 || kv_heads <= 0 || heads % kv_heads != 0 ||
      dim <= 0 || vdim <= 0 || out_stride < (int64_t)heads * vdim ||
      q_stride < (int64_t)kv_heads * dim || k_stride < (int64_t)kv_heads * dim ||
      v_stride < (int64_t)heads * vdim || gate_stride < (int64_t)heads * vdim ||
      beta_stride < heads || dt_stride < heads)
    return VLA_ERR_ARG;
  // the fewest rows per thread (8, 16, 32, 64) whose column groups fit a wave and a workgroup
  int rows = 0, split = 0;
  for (int r = 8; r <= 64; r *= 2) {
    const int sp = pow2_at_least((dim + r - 1) / r);
    if (sp <= 64 && (int64_t)sp * vdim <= 1024) {
      rows = r;
      split = sp;
      break;
    }
  }
  if (rows == 0) return VLA_ERR_HEAD_SIZE;
  const int threads = (vdim * split + 63) / 64 * 64;
  const size_t lds = (size_t)kChunk * (2 * split * rows + 2 * vdim + 5) * sizeof(float);
  if (lds > 64 * 1024) return VLA_ERR_HEAD_SIZE;
  // the rows that enter the recurrence are fp32 (the caller's projections leave them so)
  if (in_dtype != VLA_F32) return VLA_ERR_DTYPE;
  {
    return with_dtype(out_dtype, [&](auto so) {
      using SI = F32;
      using SO = decltype(so);
      using TI = typename SI::T;
      const DeltaRows<SI> in{(const TI*)q, q_stride, (const TI*)k, k_stride, (const TI*)v, v_stride,
                             (const TI*)gate, gate_stride, (const TI*)beta, beta_stride,
                             (const TI*)dt, dt_stride};
      const dim3 grid(heads, num_seqs);
      auto launch = [&](auto kernel) {
        kernel<<<grid, threads, lds, (hipStream_t)stream>>>(
            (typename SO::T*)out, out_stride, in, a_log, dt_bias, norm_weight, state,
            query_start_loc, context_lens, state_slots, heads, kv_heads, dim, vdim, split, eps);
      };
      switch (rows) {
        case 8: launch(delta_rule_kernel<SI, SO, 8>); break;
        case 16: launch(delta_rule_kernel<SI, SO, 16>); break;
        case 32: launch(delta_rule_kernel<SI, SO, 32>); break;
        default: launch(delta_rule_kernel<SI, SO, 64>); break;
      }
      VLA_SEQ_HIP_CHECK(hipGetLastError());
      return VLA_OK;
    });
  }
}
