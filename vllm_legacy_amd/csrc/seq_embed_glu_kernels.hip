// Two row-wise steps of a decoder stack over an fp32 stream.
//
// pair_hash_embed: the token's embedding row plus a row of a second table chosen by a hash of the
// previous token and the token, (prev * mul_prev + id * mul_cur) mod buckets; a sequence's first
// token takes row `buckets` (the table's last).  The previous token of a step's first row comes
// from the sequence's state slot, which a second small launch brings up to date, so a sequence may
// be cut anywhere.  The sum is fp32.
//
// clamped_glu: g = min(gate, limit), u = clamp(up, -limit, limit),
// out = g * sigmoid(alpha g) * (u + shift) on the two halves of a merged projection; fp32
// arithmetic, rows with their own strides.
#include "seq_common.h"

namespace vla {
namespace seq {
namespace {

constexpr int kThreads = 256;

template <class S>
__global__ __launch_bounds__(kThreads) void pair_hash_embed_kernel(
    float* __restrict__ out, const typename S::T* __restrict__ table,
    const typename S::T* __restrict__ pair_table, const int64_t* __restrict__ ids,
    const int64_t* __restrict__ last_token, const int* __restrict__ query_start_loc,
    const int* __restrict__ context_lens, const int* __restrict__ state_slots,
    const int* __restrict__ token_seq, int width, int vocab, int64_t buckets, int64_t mul_prev,
    int64_t mul_cur, int num_slots) {
  const int t = blockIdx.x;
  const int b = token_seq[t];
  auto token = [&](int i) {
    const int64_t id = ids[i];
    return id < 0 ? (int64_t)0 : (id >= vocab ? (int64_t)vocab - 1 : id);
  };
  const int64_t id = token(t);
  int64_t row = buckets;                         // a sequence's first token
  if (t > query_start_loc[b]) {
    row = (token(t - 1) * mul_prev + id * mul_cur) % buckets;
  } else if (context_lens[b] > 0) {
    const int slot = state_slots[b];
    int64_t prev = (unsigned)slot < (unsigned)num_slots ? last_token[slot] : 0;
    prev = prev < 0 ? 0 : (prev >= vocab ? vocab - 1 : prev);
    row = (prev * mul_prev + id * mul_cur) % buckets;
  }
  const typename S::T* e = table + id * (int64_t)width;
  const typename S::T* g = pair_table + row * (int64_t)width;
  for (int c = threadIdx.x; c < width; c += kThreads)
    out[(int64_t)t * width + c] = S::to_f32(e[c]) + S::to_f32(g[c]);
}

// after every row of the step has read its previous token
__global__ void last_token_kernel(int64_t* __restrict__ last_token, const int64_t* __restrict__ ids,
                                  const int* __restrict__ query_start_loc,
                                  const int* __restrict__ state_slots, int num_seqs, int num_slots) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= num_seqs) return;
  const int slot = state_slots[b];
  const int end = query_start_loc[b + 1];
  if ((unsigned)slot < (unsigned)num_slots && end > query_start_loc[b]) last_token[slot] = ids[end - 1];
}

__device__ __forceinline__ float clamped_glu(float gate, float up, float limit, float alpha, float shift) {
  const float g = fminf(gate, limit);
  const float u = fminf(fmaxf(up, -limit), limit);
  return g / (1.f + expf(-alpha * g)) * (u + shift);
}

template <class S>
__global__ __launch_bounds__(kThreads) void clamped_glu_kernel(
    typename S::T* __restrict__ out, int64_t out_stride, const typename S::T* __restrict__ gate,
    int64_t gate_stride, const typename S::T* __restrict__ up, int64_t up_stride, int features,
    float limit, float alpha, float shift) {
  const int64_t t = blockIdx.x;
  const int c = blockIdx.y * kThreads + threadIdx.x;
  if (c >= features) return;
  out[t * out_stride + c] = S::from_f32(clamped_glu(S::to_f32(gate[t * gate_stride + c]),
                                                    S::to_f32(up[t * up_stride + c]), limit, alpha, shift));
}

// 16-bit rows whose length is a multiple of eight and whose ends are 16-byte aligned: eight values
// per access, a workgroup per row
template <class S>
__global__ __launch_bounds__(kThreads) void clamped_glu_vec_kernel(
    typename S::T* __restrict__ out, int64_t out_stride, const typename S::T* __restrict__ gate,
    int64_t gate_stride, const typename S::T* __restrict__ up, int64_t up_stride, int features,
    float limit, float alpha, float shift) {
  const int64_t t = blockIdx.x;
  for (int c = 8 * threadIdx.x; c < features; c += 8 * kThreads) {
    const u32x4 g = *reinterpret_cast<const u32x4*>(gate + t * gate_stride + c);
    const u32x4 u = *reinterpret_cast<const u32x4*>(up + t * up_stride + c);
    u32x4 r;
#pragma unroll
    for (int e = 0; e < 4; ++e)
      r[e] = pack16<S>(clamped_glu(lo16<S>(g[e]), lo16<S>(u[e]), limit, alpha, shift),
                       clamped_glu(hi16<S>(g[e]), hi16<S>(u[e]), limit, alpha, shift));
    *reinterpret_cast<u32x4*>(out + t * out_stride + c) = r;
  }
}

}  // namespace
}  // namespace seq
}  // namespace vla

using namespace vla;
using namespace vla::seq;

extern "C" int vla_seq_pair_hash_embed(float* out, const void* table, const void* pair_table,
                                       const int64_t* ids, int64_t* last_token,
                                       const int* query_start_loc, const int* context_lens,
                                       const int* state_slots, const int* token_seq, int num_tokens,
                                       int num_seqs, int num_slots, int width, int vocab,
                                       int64_t buckets, int64_t mul_prev, int64_t mul_cur, int dtype,
                                       void* stream) {
  if (num_tokens == 0) return VLA_OK;
  if (!out || !table || !pair_table || !ids || !last_token || !query_start_loc || !context_lens ||
      !state_slots || !token_seq || num_tokens < 0 || num_seqs <= 0 || num_slots <= 0 || width <= 0 ||
      vocab <= 0 || buckets <= 0 || mul_prev < 0 || mul_cur < 0 ||
      // the hash is formed in 64-bit integers and must not wrap
      (double)vocab * ((double)mul_prev + (double)mul_cur) > 9.0e18)
    return VLA_ERR_ARG;
  const int rc = with_dtype(dtype, [&](auto s) {
    using S = decltype(s);
    using T = typename S::T;
    pair_hash_embed_kernel<S><<<num_tokens, kThreads, 0, (hipStream_t)stream>>>(
        out, (const T*)table, (const T*)pair_table, ids, last_token, query_start_loc, context_lens,
        state_slots, token_seq, width, vocab, buckets, mul_prev, mul_cur, num_slots);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
  if (rc != VLA_OK) return rc;
  last_token_kernel<<<(num_seqs + 63) / 64, 64, 0, (hipStream_t)stream>>>(
      last_token, ids, query_start_loc, state_slots, num_seqs, num_slots);
  VLA_SEQ_HIP_CHECK(hipGetLastError());
  return VLA_OK;
}

extern "C" int vla_seq_clamped_glu(void* out, int64_t out_stride, const void* gate,
                                   int64_t gate_stride, const void* up, int64_t up_stride,
                                   int num_tokens, int features, float limit, float alpha,
                                   float shift, int dtype, void* stream) {
  if (num_tokens == 0) return VLA_OK;
  if (!out || !gate || !up || num_tokens < 0 || features <= 0 || out_stride < features ||
      gate_stride < features || up_stride < features || !(limit > 0.f))
    return VLA_ERR_ARG;
  return with_dtype(dtype, [&](auto s) {
    using S = decltype(s);
    using T = typename S::T;
    if constexpr (sizeof(T) == 2) {
      const bool ok = features % 8 == 0 && ((uintptr_t)out % 16) == 0 && ((uintptr_t)gate % 16) == 0 &&
                      ((uintptr_t)up % 16) == 0 && out_stride % 8 == 0 && gate_stride % 8 == 0 &&
                      up_stride % 8 == 0;
      if (ok) {
        clamped_glu_vec_kernel<S><<<num_tokens, kThreads, 0, (hipStream_t)stream>>>(
            (T*)out, out_stride, (const T*)gate, gate_stride, (const T*)up, up_stride, features, limit,
            alpha, shift);
        VLA_SEQ_HIP_CHECK(hipGetLastError());
        return VLA_OK;
      }
    }
    clamped_glu_kernel<S><<<dim3(num_tokens, (features + kThreads - 1) / kThreads), kThreads, 0,
                            (hipStream_t)stream>>>((T*)out, out_stride, (const T*)gate, gate_stride,
                                                   (const T*)up, up_stride, features, limit, alpha,
                                                   shift);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}
