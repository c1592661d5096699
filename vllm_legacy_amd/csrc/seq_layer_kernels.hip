// Row-wise steps of decoder layers that norm a sublayer's input and its output around an fp32
// residual stream: the residual update with both norms in one launch, a short causal convolution
// over time whose last inputs live in per-sequence state slots, the side-by-side copy that feeds a
// projection of two streams, and gated / plain feed-forward activations.  One workgroup per row,
// fp32 arithmetic throughout; activations are read / written in the type the caller names.
#include "seq_common.h"

namespace vla {
namespace seq {
namespace {

constexpr int kThreads = 256;
constexpr int kKeep = 8;          // row elements a thread keeps in registers (rows up to 2048)
constexpr int kMaxTaps = 32;

template <class SY, class SO>
__global__ __launch_bounds__(kThreads) void residual_norms_kernel(
    float* __restrict__ x, const typename SY::T* __restrict__ y, int64_t y_stride,
    const float* __restrict__ y_bias, const float* __restrict__ post_w,
    const float* __restrict__ layer_scale,
    const float* __restrict__ add_row, typename SO::T* __restrict__ out,
    const float* __restrict__ pre_w, float eps, int width) {
  __shared__ float red[16];
  const int64_t base = (int64_t)blockIdx.x * width;
  float keep[kKeep], keepx[kKeep];
  float inv_y = 0.f;
  // the stream's row is asked for before the first reduction, so its latency hides behind it
#pragma unroll
  for (int i = 0; i < kKeep; ++i) {
    const int c = threadIdx.x + i * kThreads;
    keepx[i] = c < width ? x[base + c] : 0.f;
  }
  if (y != nullptr) {
    const typename SY::T* yr = y + (int64_t)blockIdx.x * y_stride;
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < kKeep; ++i) {
      const int c = threadIdx.x + i * kThreads;
      if (c < width) {
        keep[i] = SY::to_f32(yr[c]) + (y_bias != nullptr ? y_bias[c] : 0.f);
        ss += keep[i] * keep[i];
      }
    }
    for (int c = threadIdx.x + kKeep * kThreads; c < width; c += kThreads) {
      const float v = SY::to_f32(yr[c]) + (y_bias != nullptr ? y_bias[c] : 0.f);
      ss += v * v;
    }
    ss = block_sum(ss, red);
    inv_y = 1.f / sqrtf(ss / (float)width + eps);
  }
  const bool writes = y != nullptr || add_row != nullptr;
  float ss = 0.f;
  auto update = [&](int c, float xv, float yv) {
    float v = xv;
    if (y != nullptr) {
      float u = yv * inv_y * post_w[c];
      if (layer_scale != nullptr) u *= layer_scale[c];
      v += u;
    }
    if (add_row != nullptr) v += add_row[c];
    if (writes) x[base + c] = v;
    ss += v * v;
    return v;
  };
#pragma unroll
  for (int i = 0; i < kKeep; ++i) {
    const int c = threadIdx.x + i * kThreads;
    if (c < width) keep[i] = update(c, keepx[i], y != nullptr ? keep[i] : 0.f);
  }
  for (int c = threadIdx.x + kKeep * kThreads; c < width; c += kThreads)
    update(c, x[base + c], y != nullptr ? SY::to_f32(y[(int64_t)blockIdx.x * y_stride + c]) +
                                              (y_bias != nullptr ? y_bias[c] : 0.f)
                                        : 0.f);
  if (out == nullptr) return;
  if (pre_w == nullptr) {           // no norm ahead of the reader: the stream's row as it is
#pragma unroll
    for (int i = 0; i < kKeep; ++i) {
      const int c = threadIdx.x + i * kThreads;
      if (c < width) out[base + c] = SO::from_f32(keep[i]);
    }
    for (int c = threadIdx.x + kKeep * kThreads; c < width; c += kThreads)
      out[base + c] = SO::from_f32(x[base + c]);
    return;
  }
  ss = block_sum(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)width + eps);
#pragma unroll
  for (int i = 0; i < kKeep; ++i) {
    const int c = threadIdx.x + i * kThreads;
    if (c < width) out[base + c] = SO::from_f32(keep[i] * inv * pre_w[c]);
  }
  for (int c = threadIdx.x + kKeep * kThreads; c < width; c += kThreads)
    out[base + c] = SO::from_f32(x[base + c] * inv * pre_w[c]);
}

// out[t] = h[t] + sum_d w[:, taps - 1 - d] * h at position p - d; rows of earlier steps come from
// the state slot, positions before the sequence's start are zeros.
template <class S>
__global__ __launch_bounds__(kThreads) void causal_conv_kernel(
    typename S::T* __restrict__ out, const float* __restrict__ h, const float* __restrict__ w,
    const float* __restrict__ state, const int* __restrict__ query_start_loc,
    const int* __restrict__ context_lens, const int* __restrict__ state_slots,
    const int* __restrict__ token_seq, int width, int taps) {
  const int t = blockIdx.x;
  const int b = token_seq[t];
  const int start = query_start_loc[b], ctx = context_lens[b];
  const int p = ctx + (t - start);
  const float* st = state + (int64_t)state_slots[b] * (taps - 1) * width;
  for (int c = threadIdx.x; c < width; c += kThreads) {
    const float cur = h[(int64_t)t * width + c];
    float acc = cur;
    for (int d = 0; d < taps; ++d) {
      const int s = p - d;
      if (s < 0) break;
      float v;
      if (s >= ctx)
        v = d == 0 ? cur : h[(int64_t)(t - d) * width + c];
      else
        v = st[(int64_t)(s - ctx + taps - 1) * width + c];
      acc += w[(int64_t)c * taps + (taps - 1 - d)] * v;
    }
    out[(int64_t)t * width + c] = S::from_f32(acc);
  }
}

// The last taps - 1 inputs of every sequence of the step, oldest first.  A thread owns a channel:
// it reads what it keeps of the old state before it writes.
__global__ __launch_bounds__(kThreads) void causal_conv_state_kernel(
    float* __restrict__ state, const float* __restrict__ h, const int* __restrict__ query_start_loc,
    const int* __restrict__ context_lens, const int* __restrict__ state_slots, int width, int taps) {
  const int b = blockIdx.y;
  const int c = blockIdx.x * kThreads + threadIdx.x;
  if (c >= width) return;
  const int start = query_start_loc[b], n = query_start_loc[b + 1] - start, ctx = context_lens[b];
  float* st = state + (int64_t)state_slots[b] * (taps - 1) * width;
  float keep[kMaxTaps];
  for (int i = 0; i < taps - 1; ++i) {
    const int s = ctx + n - (taps - 1) + i;     // position that lands in entry i
    float v = 0.f;
    if (s >= ctx)
      v = h[(int64_t)(start + s - ctx) * width + c];
    else if (s >= 0)
      v = st[(int64_t)(s - ctx + taps - 1) * width + c];
    keep[i] = v;
  }
  for (int i = 0; i < taps - 1; ++i) st[(int64_t)i * width + c] = keep[i];
}

template <class S>
__global__ __launch_bounds__(kThreads) void concat_cast_kernel(typename S::T* __restrict__ out,
                                                              const float* __restrict__ a,
                                                              const float* __restrict__ b, int width) {
  const int64_t t = blockIdx.x;
  for (int c = threadIdx.x; c < width; c += kThreads) {
    out[t * 2 * width + c] = S::from_f32(a[t * width + c]);
    out[t * 2 * width + width + c] = S::from_f32(b[t * width + c]);
  }
}

__device__ __forceinline__ float activate(float z, int act) {
  switch (act) {
    case VLA_ACT_RELU: return fmaxf(z, 0.f);
    case VLA_ACT_RELU2: {
      const float r = fmaxf(z, 0.f);
      return r * r;
    }
    case VLA_ACT_SILU: return z / (1.f + expf(-z));
    default: return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
  }
}

// out = act(gate) * up (up null: act(gate)), rows with their own strides
template <class S>
__global__ __launch_bounds__(kThreads) void gated_act_kernel(
    typename S::T* __restrict__ out, int64_t out_stride, const typename S::T* __restrict__ gate,
    int64_t gate_stride, const typename S::T* __restrict__ up, int64_t up_stride, int features,
    int act) {
  const int64_t t = blockIdx.x;
  const int c = blockIdx.y * kThreads + threadIdx.x;
  if (c >= features) return;
  float v = activate(S::to_f32(gate[t * gate_stride + c]), act);
  if (up != nullptr) v *= S::to_f32(up[t * up_stride + c]);
  out[t * out_stride + c] = S::from_f32(v);
}

// 16-bit rows whose length is a multiple of eight and whose ends are 16-byte aligned: eight values
// per access, a workgroup per row
template <class S>
__global__ __launch_bounds__(kThreads) void gated_act_vec_kernel(
    typename S::T* __restrict__ out, int64_t out_stride, const typename S::T* __restrict__ gate,
    int64_t gate_stride, const typename S::T* __restrict__ up, int64_t up_stride, int features,
    int act) {
  const int64_t t = blockIdx.x;
  for (int c = 8 * threadIdx.x; c < features; c += 8 * kThreads) {
    const u32x4 g = *reinterpret_cast<const u32x4*>(gate + t * gate_stride + c);
    u32x4 u = {0u, 0u, 0u, 0u};
    if (up != nullptr) u = *reinterpret_cast<const u32x4*>(up + t * up_stride + c);
    u32x4 r;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float a = activate(lo16<S>(g[e]), act), b = activate(hi16<S>(g[e]), act);
      if (up != nullptr) {
        a *= lo16<S>(u[e]);
        b *= hi16<S>(u[e]);
      }
      r[e] = pack16<S>(a, b);
    }
    *reinterpret_cast<u32x4*>(out + t * out_stride + c) = r;
  }
}

template <class F>
int with_two_dtypes(int a, int b, F&& f) {
  return with_dtype(a, [&](auto sa) { return with_dtype(b, [&](auto sb) { return f(sa, sb); }); });
}

}  // namespace
}  // namespace seq
}  // namespace vla

using namespace vla;
using namespace vla::seq;

extern "C" int vla_seq_residual_norms(float* x, const void* y, int64_t y_stride, int y_dtype,
                                      const float* y_bias, const float* post_weight,
                                      const float* layer_scale,
                                      const float* add_row, void* out, const float* pre_weight,
                                      float eps, int num_tokens, int width, int out_dtype,
                                      void* stream) {
  if (num_tokens == 0) return VLA_OK;
  if (!x || num_tokens < 0 || width <= 0 || (y && (!post_weight || y_stride < width)))
    return VLA_ERR_ARG;
  return with_two_dtypes(y ? y_dtype : VLA_F32, out ? out_dtype : VLA_F32, [&](auto sy, auto so) {
    using SY = decltype(sy);
    using SO = decltype(so);
    residual_norms_kernel<SY, SO><<<num_tokens, kThreads, 0, (hipStream_t)stream>>>(
        x, (const typename SY::T*)y, y_stride, y_bias, post_weight, layer_scale, add_row,
        (typename SO::T*)out, pre_weight, eps, width);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}

extern "C" int vla_seq_causal_conv(void* out, const float* h, const float* weight, float* state,
                                   const int* query_start_loc, const int* context_lens,
                                   const int* state_slots, const int* token_seq, int num_tokens,
                                   int num_seqs, int num_slots, int width, int taps, int dtype,
                                   void* stream) {
  if (num_tokens == 0) return VLA_OK;
  if (!out || !h || !weight || !query_start_loc || !context_lens || !state_slots || !token_seq ||
      num_tokens < 0 || num_seqs <= 0 || width <= 0 || taps < 1 || taps > kMaxTaps ||
      (taps > 1 && (!state || num_slots <= 0)))
    return VLA_ERR_ARG;
  const int rc = with_dtype(dtype, [&](auto s) {
    using S = decltype(s);
    causal_conv_kernel<S><<<num_tokens, kThreads, 0, (hipStream_t)stream>>>(
        (typename S::T*)out, h, weight, state, query_start_loc, context_lens, state_slots, token_seq,
        width, taps);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
  if (rc != VLA_OK || taps == 1) return rc;
  causal_conv_state_kernel<<<dim3((width + kThreads - 1) / kThreads, num_seqs), kThreads, 0,
                             (hipStream_t)stream>>>(state, h, query_start_loc, context_lens,
                                                    state_slots, width, taps);
  VLA_SEQ_HIP_CHECK(hipGetLastError());
  return VLA_OK;
}

extern "C" int vla_seq_concat_cast(void* out, const float* a, const float* b, int num_tokens,
                                   int width, int dtype, void* stream) {
  if (num_tokens == 0) return VLA_OK;
  if (!out || !a || !b || num_tokens < 0 || width <= 0) return VLA_ERR_ARG;
  return with_dtype(dtype, [&](auto s) {
    using S = decltype(s);
    concat_cast_kernel<S><<<num_tokens, kThreads, 0, (hipStream_t)stream>>>((typename S::T*)out, a, b,
                                                                          width);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}

extern "C" int vla_seq_gated_act(void* out, int64_t out_stride, const void* gate,
                                 int64_t gate_stride, const void* up, int64_t up_stride,
                                 int num_tokens, int features, int act, int dtype, void* stream) {
  if (num_tokens == 0) return VLA_OK;
  if (!out || !gate || num_tokens < 0 || features <= 0 || out_stride < features ||
      gate_stride < features || (up && up_stride < features) || act < VLA_ACT_RELU ||
      act > VLA_ACT_GELU_TANH)
    return VLA_ERR_ARG;
  return with_dtype(dtype, [&](auto s) {
    using S = decltype(s);
    if constexpr (sizeof(typename S::T) == 2) {
      const bool ok = features % 8 == 0 && ((uintptr_t)out % 16) == 0 && ((uintptr_t)gate % 16) == 0 &&
                      (!up || ((uintptr_t)up % 16) == 0) && out_stride % 8 == 0 &&
                      gate_stride % 8 == 0 && (!up || up_stride % 8 == 0);
      if (ok) {
        gated_act_vec_kernel<S><<<num_tokens, kThreads, 0, (hipStream_t)stream>>>(
            (typename S::T*)out, out_stride, (const typename S::T*)gate, gate_stride,
            (const typename S::T*)up, up_stride, features, act);
        VLA_SEQ_HIP_CHECK(hipGetLastError());
        return VLA_OK;
      }
    }
    gated_act_kernel<S><<<dim3(num_tokens, (features + kThreads - 1) / kThreads), kThreads, 0,
                          (hipStream_t)stream>>>((typename S::T*)out, out_stride,
                                                 (const typename S::T*)gate, gate_stride,
                                                 (const typename S::T*)up, up_stride, features, act);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}
