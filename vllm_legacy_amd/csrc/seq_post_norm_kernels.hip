// Row-wise steps of decoder layers that norm the stream itself after every sublayer (the norm
// follows the sum, so the fp32 stream is what the next sublayer reads):
//   post_norm         x <- N(alpha x + y) * w, and a copy of the new x in the activation dtype
//   rms_norm_rows     plain RMS norm of projected rows (a latent before its up-projection)
//   short_conv        causal convolution over time per channel with bias and activation, the last
//                     taps - 1 inputs of every sequence in state slots
//   gated_act_lookup  act(gate) * table[id, columns]: a per-token embedding gates a projection
//   embed_scaled      table[id] * scale as the fp32 stream
//   softcap           z <- cap * tanh(z / cap)
// One workgroup per row, fp32 arithmetic throughout; rows are read / written in the types named.
#include "seq_common.h"

namespace vla {
namespace seq {
namespace {

constexpr int kThreads = 256;
constexpr int kKeep = 8;          // row elements a thread keeps in registers (rows up to 2048)
constexpr int kMaxTaps = 32;

__device__ __forceinline__ float activate(float z, int act) {
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

template <class SY, class SO>
__global__ __launch_bounds__(kThreads) void post_norm_kernel(
    float* __restrict__ x, float alpha, const typename SY::T* __restrict__ y, int64_t y_stride,
    const float* __restrict__ weight, float eps, typename SO::T* __restrict__ out, int width) {
  __shared__ float red[16];
  const int64_t base = (int64_t)blockIdx.x * width;
  const typename SY::T* yr = y + (int64_t)blockIdx.x * y_stride;
  float keep[kKeep];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < kKeep; ++i) {
    const int c = threadIdx.x + i * kThreads;
    keep[i] = 0.f;
    if (c < width) {
      keep[i] = alpha * x[base + c] + SY::to_f32(yr[c]);
      ss += keep[i] * keep[i];
    }
  }
  for (int c = threadIdx.x + kKeep * kThreads; c < width; c += kThreads) {
    const float v = alpha * x[base + c] + SY::to_f32(yr[c]);
    x[base + c] = v;                // parked in the stream until the scale is known
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)width + eps);
#pragma unroll
  for (int i = 0; i < kKeep; ++i) {
    const int c = threadIdx.x + i * kThreads;
    if (c < width) {
      const float v = keep[i] * inv * weight[c];
      x[base + c] = v;
      if (out != nullptr) out[base + c] = SO::from_f32(v);
    }
  }
  for (int c = threadIdx.x + kKeep * kThreads; c < width; c += kThreads) {
    const float v = x[base + c] * inv * weight[c];
    x[base + c] = v;
    if (out != nullptr) out[base + c] = SO::from_f32(v);
  }
}

template <class SI, class SO>
__global__ __launch_bounds__(kThreads) void rms_norm_rows_kernel(
    typename SO::T* __restrict__ out, int64_t out_stride, const typename SI::T* __restrict__ in,
    int64_t in_stride, const float* __restrict__ weight, float eps, int n) {
  __shared__ float red[16];
  const typename SI::T* r = in + (int64_t)blockIdx.x * in_stride;
  float ss = 0.f;
  for (int c = threadIdx.x; c < n; c += kThreads) {
    const float v = SI::to_f32(r[c]);
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)n + eps);
  for (int c = threadIdx.x; c < n; c += kThreads)
    out[(int64_t)blockIdx.x * out_stride + c] = SO::from_f32(SI::to_f32(r[c]) * inv * weight[c]);
}

// out[t, c] = act(bias[c] + sum_d w[c, taps - 1 - d] * u at position p - d); rows of earlier
// steps come from the state slot, positions before the sequence's start are zeros.
template <class SI, class SO>
__global__ __launch_bounds__(kThreads) void short_conv_kernel(
    typename SO::T* __restrict__ out, int64_t out_stride, const typename SI::T* __restrict__ u,
    int64_t u_stride, const float* __restrict__ w, const float* __restrict__ bias,
    const float* __restrict__ state, const int* __restrict__ query_start_loc,
    const int* __restrict__ context_lens, const int* __restrict__ state_slots,
    const int* __restrict__ token_seq, int channels, int taps, int act) {
  const int t = blockIdx.x;
  const int b = token_seq[t];
  const int start = query_start_loc[b], ctx = context_lens[b];
  const int p = ctx + (t - start);
  const float* st = state + (int64_t)state_slots[b] * (taps - 1) * channels;
  for (int c = threadIdx.x; c < channels; c += kThreads) {
    float acc = bias != nullptr ? bias[c] : 0.f;
    for (int d = 0; d < taps; ++d) {
      const int s = p - d;
      if (s < 0) break;
      const float v = s >= ctx ? SI::to_f32(u[(int64_t)(t - d) * u_stride + c])
                               : st[(int64_t)(s - ctx + taps - 1) * channels + c];
      acc += w[(int64_t)c * taps + (taps - 1 - d)] * v;
    }
    out[(int64_t)t * out_stride + c] = SO::from_f32(activate(acc, act));
  }
}

// The last taps - 1 inputs of every sequence of the step, oldest first.  A thread owns a channel:
// it reads what it keeps of the old state before it writes.
template <class SI>
__global__ __launch_bounds__(kThreads) void short_conv_state_kernel(
    float* __restrict__ state, const typename SI::T* __restrict__ u, int64_t u_stride,
    const int* __restrict__ query_start_loc, const int* __restrict__ context_lens,
    const int* __restrict__ state_slots, int channels, int taps) {
  const int b = blockIdx.y;
  const int c = blockIdx.x * kThreads + threadIdx.x;
  if (c >= channels) return;
  const int start = query_start_loc[b], n = query_start_loc[b + 1] - start, ctx = context_lens[b];
  float* st = state + (int64_t)state_slots[b] * (taps - 1) * channels;
  float keep[kMaxTaps];
  for (int i = 0; i < taps - 1; ++i) {
    const int s = ctx + n - (taps - 1) + i;     // position that lands in entry i
    float v = 0.f;
    if (s >= ctx)
      v = SI::to_f32(u[(int64_t)(start + s - ctx) * u_stride + c]);
    else if (s >= 0)
      v = st[(int64_t)(s - ctx + taps - 1) * channels + c];
    keep[i] = v;
  }
  for (int i = 0; i < taps - 1; ++i) st[(int64_t)i * channels + c] = keep[i];
}

template <class SI, class ST, class SO>
__global__ __launch_bounds__(kThreads) void gated_act_lookup_kernel(
    typename SO::T* __restrict__ out, int64_t out_stride, const typename SI::T* __restrict__ gate,
    int64_t gate_stride, const typename ST::T* __restrict__ table, int64_t table_stride,
    const int64_t* __restrict__ ids, int rows, int first_col, int features, int act) {
  const int64_t t = blockIdx.x;
  int64_t id = ids[t];
  id = id < 0 ? 0 : (id >= rows ? rows - 1 : id);
  for (int c = threadIdx.x; c < features; c += kThreads)
    out[t * out_stride + c] = SO::from_f32(activate(SI::to_f32(gate[t * gate_stride + c]), act) *
                                           ST::to_f32(table[id * table_stride + first_col + c]));
}

template <class S>
__global__ __launch_bounds__(kThreads) void embed_scaled_kernel(
    float* __restrict__ out, const typename S::T* __restrict__ table, const int64_t* __restrict__ ids,
    float scale, int width, int vocab) {
  const int t = blockIdx.x;
  int64_t id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const typename S::T* row = table + id * (int64_t)width;
  for (int c = threadIdx.x; c < width; c += kThreads)
    out[(int64_t)t * width + c] = S::to_f32(row[c]) * scale;
}

__global__ __launch_bounds__(kThreads) void softcap_kernel(float* __restrict__ z, int64_t n, float cap) {
  const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i < n) z[i] = cap * tanhf(z[i] / cap);
}

template <class F>
int with_two(int a, int b, F&& f) {
  return with_dtype(a, [&](auto sa) { return with_dtype(b, [&](auto sb) { return f(sa, sb); }); });
}

}  // namespace
}  // namespace seq
}  // namespace vla

using namespace vla;
using namespace vla::seq;

extern "C" int vla_seq_post_norm(float* x, float alpha, const void* y, int64_t y_stride, int y_dtype,
                                 const float* weight, float eps, void* out, int out_dtype,
                                 int num_tokens, int width, void* stream) {
  if (num_tokens == 0) return VLA_OK;
  if (!x || !y || !weight || num_tokens < 0 || width <= 0 || y_stride < width) return VLA_ERR_ARG;
  return with_two(y_dtype, out ? out_dtype : VLA_F32, [&](auto sy, auto so) {
    using SY = decltype(sy);
    using SO = decltype(so);
    post_norm_kernel<SY, SO><<<num_tokens, kThreads, 0, (hipStream_t)stream>>>(
        x, alpha, (const typename SY::T*)y, y_stride, weight, eps, (typename SO::T*)out, width);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}

extern "C" int vla_seq_rms_norm_rows(void* out, int64_t out_stride, int out_dtype, const void* in,
                                     int64_t in_stride, int in_dtype, const float* weight, float eps,
                                     int num_tokens, int n, void* stream) {
  if (num_tokens == 0) return VLA_OK;
  if (!out || !in || !weight || num_tokens < 0 || n <= 0 || out_stride < n || in_stride < n)
    return VLA_ERR_ARG;
  return with_two(in_dtype, out_dtype, [&](auto si, auto so) {
    using SI = decltype(si);
    using SO = decltype(so);
    rms_norm_rows_kernel<SI, SO><<<num_tokens, kThreads, 0, (hipStream_t)stream>>>(
        (typename SO::T*)out, out_stride, (const typename SI::T*)in, in_stride, weight, eps, n);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}

extern "C" int vla_seq_short_conv(void* out, int64_t out_stride, int out_dtype, const void* u,
                                  int64_t u_stride, int u_dtype, const float* weight,
                                  const float* bias, float* state, const int* query_start_loc,
                                  const int* context_lens, const int* state_slots,
                                  const int* token_seq, int num_tokens, int num_seqs, int num_slots,
                                  int channels, int taps, int act, void* stream) {
  if (num_tokens == 0) return VLA_OK;
  if (!out || !u || !weight || !query_start_loc || !context_lens || !state_slots || !token_seq ||
      num_tokens < 0 || num_seqs <= 0 || num_seqs > 65535 || channels <= 0 || taps < 1 ||
      taps > kMaxTaps || out_stride < channels || u_stride < channels || act < VLA_ACT_NONE ||
      act > VLA_ACT_GELU_TANH || (taps > 1 && (!state || num_slots <= 0)))
    return VLA_ERR_ARG;
  return with_two(u_dtype, out_dtype, [&](auto si, auto so) {
    using SI = decltype(si);
    using SO = decltype(so);
    short_conv_kernel<SI, SO><<<num_tokens, kThreads, 0, (hipStream_t)stream>>>(
        (typename SO::T*)out, out_stride, (const typename SI::T*)u, u_stride, weight, bias, state,
        query_start_loc, context_lens, state_slots, token_seq, channels, taps, act);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    if (taps > 1) {
      short_conv_state_kernel<SI><<<dim3((channels + kThreads - 1) / kThreads, num_seqs), kThreads, 0,
                                    (hipStream_t)stream>>>(state, (const typename SI::T*)u, u_stride,
                                                           query_start_loc, context_lens, state_slots,
                                                           channels, taps);
      VLA_SEQ_HIP_CHECK(hipGetLastError());
    }
    return VLA_OK;
  });
}

extern "C" int vla_seq_gated_act_lookup(void* out, int64_t out_stride, int out_dtype,
                                        const void* gate, int64_t gate_stride, int gate_dtype,
                                        const void* table, int64_t table_stride, int table_dtype,
                                        const int64_t* ids, int rows, int first_col, int num_tokens,
                                        int features, int act, void* stream) {
  if (num_tokens == 0) return VLA_OK;
  if (!out || !gate || !table || !ids || num_tokens < 0 || features <= 0 || rows <= 0 ||
      first_col < 0 || out_stride < features || gate_stride < features ||
      table_stride < (int64_t)first_col + features || act < VLA_ACT_NONE || act > VLA_ACT_GELU_TANH)
    return VLA_ERR_ARG;
  return with_two(gate_dtype, out_dtype, [&](auto si, auto so) {
    return with_dtype(table_dtype, [&](auto st) {
      using SI = decltype(si);
      using SO = decltype(so);
      using ST = decltype(st);
      gated_act_lookup_kernel<SI, ST, SO><<<num_tokens, kThreads, 0, (hipStream_t)stream>>>(
          (typename SO::T*)out, out_stride, (const typename SI::T*)gate, gate_stride,
          (const typename ST::T*)table, table_stride, ids, rows, first_col, features, act);
      VLA_SEQ_HIP_CHECK(hipGetLastError());
      return VLA_OK;
    });
  });
}

extern "C" int vla_seq_embed_scaled(float* out, const void* table, const int64_t* ids, float scale,
                                    int num_tokens, int width, int vocab, int dtype, void* stream) {
  if (num_tokens == 0) return VLA_OK;
  if (!out || !table || !ids || num_tokens < 0 || width <= 0 || vocab <= 0) return VLA_ERR_ARG;
  return with_dtype(dtype, [&](auto s) {
    using S = decltype(s);
    embed_scaled_kernel<S><<<num_tokens, kThreads, 0, (hipStream_t)stream>>>(
        out, (const typename S::T*)table, ids, scale, width, vocab);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}

extern "C" int vla_seq_softcap(float* z, int64_t n, float cap, void* stream) {
  if (n == 0) return VLA_OK;
  if (!z || n < 0 || !(cap > 0.f)) return VLA_ERR_ARG;
  softcap_kernel<<<(unsigned)((n + kThreads - 1) / kThreads), kThreads, 0, (hipStream_t)stream>>>(z, n, cap);
  VLA_SEQ_HIP_CHECK(hipGetLastError());
  return VLA_OK;
}
