// Element-wise gated recurrences: every channel carries one fp32 number per sequence,
//   S_t = a_t S_(t-1) + b_t,
// where a_t and b_t come from the current token alone.  minGRU:
//   a = 1 - z, b = z c,   z = sigmoid(zp),   c = up + 1/2 (up >= 0), sigmoid(up) (up < 0),
//   out_t = S_t * silu(gp),
// with zp, up and gp projections of the token.  The real-gated linear recurrent unit:
//   a = exp(-rate sigmoid(r)),  b = sqrt(1 - a^2) sigmoid(i) u,   out_t = S_t * gelu_tanh(y).  The state lives in slots
// [num_slots, channels]; a sequence whose context length is 0 starts from zero whatever its slot
// held.  Gates, candidate and state are fp32; the projections come in the activation dtype.
//
// Short runs of rows (decode steps, small portions): one thread per (sequence, channel) walks the
// run.  Long runs are cut into pieces of kPiece rows that are walked at the same time: the
// recurrence is linear in S, so a piece is summed up by (A, B) with S_end = A S_start + B; a second
// launch chains the pieces' sums into the state each piece starts from (and leaves the run's last
// state in the slot), a third walks every piece again from its true start and writes the outputs.
#include "seq_common.h"

namespace vla {
namespace seq {
namespace {

constexpr int kThreads = 256;
constexpr int kPiece = 128;

__device__ __forceinline__ float sigmoidf(float v) { return 1.f / (1.f + expf(-v)); }
__device__ __forceinline__ float candidate(float u) { return u >= 0.f ? u + 0.5f : sigmoidf(u); }

// A recurrence S_t = a_t S_(t-1) + b_t per channel is given by a gate type G:
//   G::In            what a row holds for a channel
//   load(t, c, w)    reads it (w: also what only the output needs)
//   advance(in, s, a)  returns a_t s + b_t and multiplies a by a_t
//   store(t, c, in, s) writes the row's output from the new state

template <class S>
struct MinGRUGate {
  const typename S::T* zp;
  int64_t z_stride;
  const typename S::T* up;
  int64_t u_stride;
  const typename S::T* gp;
  int64_t g_stride;
  typename S::T* out;
  int64_t out_stride;
  struct In {
    float z, u, g;
  };
  __device__ __forceinline__ In load(int64_t t, int c, bool w) const {
    In in;
    in.z = S::to_f32(zp[t * z_stride + c]);
    in.u = S::to_f32(up[t * u_stride + c]);
    in.g = w ? S::to_f32(gp[t * g_stride + c]) : 0.f;
    return in;
  }
  __device__ __forceinline__ float advance(const In& in, float s, float& a) const {
    const float zz = sigmoidf(in.z);
    a *= 1.f - zz;
    return (1.f - zz) * s + zz * candidate(in.u);
  }
  __device__ __forceinline__ void store(int64_t t, int c, const In& in, float s) const {
    out[t * out_stride + c] = S::from_f32(s * (in.g * sigmoidf(in.g)));
  }
};

// Real-gated linear recurrent unit: a = exp(-rate * sigmoid(r)), b = sqrt(1 - a^2) sigmoid(i) u,
// output S * gelu_tanh(y); r, i the gates' products, u the recurrent branch, y the other branch
// before its activation (fp32 rows), rate fp32 per channel.
template <class S>
struct RGLRUGate {
  const float* rp;
  int64_t r_stride;
  const float* ip;
  int64_t i_stride;
  const float* up;
  int64_t u_stride;
  const float* yp;
  int64_t y_stride;
  const float* rate;
  typename S::T* out;
  int64_t out_stride;
  int gate_block;             // the gates' rows come in blocks of this many channels,
  int64_t gate_block_stride;  // this far apart (blocks of a batched product)
  struct In {
    float r, i, u, y, rate;
  };
  __device__ __forceinline__ In load(int64_t t, int c, bool w) const {
    In in;
    const int64_t gc = (int64_t)(c / gate_block) * gate_block_stride + c % gate_block;
    in.r = rp[t * r_stride + gc];
    in.i = ip[t * i_stride + gc];
    in.u = up[t * u_stride + c];
    in.y = w ? yp[t * y_stride + c] : 0.f;
    in.rate = rate[c];
    return in;
  }
  __device__ __forceinline__ float advance(const In& in, float s, float& a) const {
    const float log_a = -in.rate * sigmoidf(in.r);
    const float at = expf(log_a);
    a *= at;
    // 1 - a^2 without the cancellation near a = 1
    return at * s + sqrtf(-expm1f(2.f * log_a)) * (sigmoidf(in.i) * in.u);
  }
  __device__ __forceinline__ void store(int64_t t, int c, const In& in, float s) const {
    const float z = in.y;
    const float act = 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
    out[t * out_stride + c] = S::from_f32(s * act);
  }
};

// walks rows [r0, r1) of channel c from state s; writes outputs when WRITE; returns the state
template <class G, bool WRITE>
__device__ __forceinline__ float walk(const G& r, int r0, int r1, int c, float s, float* decay) {
  float a = 1.f;
  constexpr int U = 4;
  int t = r0;
  for (; t + U <= r1; t += U) {
    typename G::In in[U];
#pragma unroll
    for (int i = 0; i < U; ++i) in[i] = r.load(t + i, c, WRITE);
#pragma unroll
    for (int i = 0; i < U; ++i) {
      s = r.advance(in[i], s, a);
      if (WRITE) r.store(t + i, c, in[i], s);
    }
  }
  for (; t < r1; ++t) {
    const typename G::In in = r.load(t, c, WRITE);
    s = r.advance(in, s, a);
    if (WRITE) r.store(t, c, in, s);
  }
  if (decay != nullptr) *decay = a;
  return s;
}

template <class G>
__global__ __launch_bounds__(kThreads) void gated_walk_kernel(
    G r, float* __restrict__ state, const int* __restrict__ query_start_loc,
    const int* __restrict__ context_lens, const int* __restrict__ state_slots, int channels) {
  const int b = blockIdx.y;
  const int c = blockIdx.x * kThreads + threadIdx.x;
  if (c >= channels) return;
  float* st = state + (int64_t)state_slots[b] * channels + c;
  const float s0 = context_lens[b] > 0 ? *st : 0.f;
  *st = walk<G, true>(r, query_start_loc[b], query_start_loc[b + 1], c, s0, nullptr);
}

// sums[b][piece][0 / 1][c] = (A, B) of the piece walked from zero
template <class G>
__global__ __launch_bounds__(kThreads) void gated_piece_sums_kernel(
    G r, float* __restrict__ sums, const int* __restrict__ query_start_loc, int channels,
    int max_pieces) {
  const int b = blockIdx.z, piece = blockIdx.y;
  const int c = blockIdx.x * kThreads + threadIdx.x;
  const int start = query_start_loc[b] + piece * kPiece, end = query_start_loc[b + 1];
  if (c >= channels || start >= end) return;
  float a;
  const float s = walk<G, false>(r, start, min(end, start + kPiece), c, 0.f, &a);
  float* dst = sums + (((int64_t)b * max_pieces + piece) * 2) * channels + c;
  dst[0] = a;
  dst[channels] = s;
}

// sums[b][piece][0][c] <- the state the piece starts from; the slot gets the run's last state
__global__ __launch_bounds__(kThreads) void gated_chain_kernel(
    float* __restrict__ sums, float* __restrict__ state, const int* __restrict__ query_start_loc,
    const int* __restrict__ context_lens, const int* __restrict__ state_slots, int channels,
    int max_pieces) {
  const int b = blockIdx.y;
  const int c = blockIdx.x * kThreads + threadIdx.x;
  if (c >= channels) return;
  const int n = query_start_loc[b + 1] - query_start_loc[b];
  const int pieces = (n + kPiece - 1) / kPiece;
  float* st = state + (int64_t)state_slots[b] * channels + c;
  float s = context_lens[b] > 0 ? *st : 0.f;
  for (int i = 0; i < pieces; ++i) {
    float* e = sums + (((int64_t)b * max_pieces + i) * 2) * channels + c;
    const float a = e[0], add = e[channels];
    e[0] = s;
    s = a * s + add;
  }
  *st = s;
}

template <class G>
__global__ __launch_bounds__(kThreads) void gated_piece_walk_kernel(
    G r, const float* __restrict__ sums, const int* __restrict__ query_start_loc,
    int channels, int max_pieces) {
  const int b = blockIdx.z, piece = blockIdx.y;
  const int c = blockIdx.x * kThreads + threadIdx.x;
  const int start = query_start_loc[b] + piece * kPiece, end = query_start_loc[b + 1];
  if (c >= channels || start >= end) return;
  const float s0 = sums[(((int64_t)b * max_pieces + piece) * 2) * channels + c];
  walk<G, true>(r, start, min(end, start + kPiece), c, s0, nullptr);
}

// One launch for short runs; three (sums of the pieces, their chain, the pieces again) for long
// ones when the caller brought scratch.
template <class G>
int run_gated_scan(const G& r, float* state, const int* query_start_loc, const int* context_lens,
                   const int* state_slots, int num_seqs, int max_query_len, int channels,
                   float* scratch, int64_t scratch_floats, hipStream_t st) {
  const int64_t need = vla_seq_mingru_scratch_floats(num_seqs, max_query_len, channels);
  const bool pieces = need > 0 && scratch != nullptr && scratch_floats >= need;
  const int max_pieces = (max_query_len + kPiece - 1) / kPiece;
  if (pieces && max_pieces > 65535) return VLA_ERR_ARG;
  const int cb = (channels + kThreads - 1) / kThreads;
  if (!pieces) {
    gated_walk_kernel<G><<<dim3(cb, num_seqs), kThreads, 0, st>>>(r, state, query_start_loc, context_lens,
                                                                  state_slots, channels);
  } else {
    gated_piece_sums_kernel<G><<<dim3(cb, max_pieces, num_seqs), kThreads, 0, st>>>(
        r, scratch, query_start_loc, channels, max_pieces);
    gated_chain_kernel<<<dim3(cb, num_seqs), kThreads, 0, st>>>(
        scratch, state, query_start_loc, context_lens, state_slots, channels, max_pieces);
    gated_piece_walk_kernel<G><<<dim3(cb, max_pieces, num_seqs), kThreads, 0, st>>>(
        r, scratch, query_start_loc, channels, max_pieces);
  }
  VLA_SEQ_HIP_CHECK(hipGetLastError());
  return VLA_OK;
}

}  // namespace
}  // namespace seq
}  // namespace vla

using namespace vla;
using namespace vla::seq;

extern "C" int64_t vla_seq_mingru_scratch_floats(int num_seqs, int max_query_len, int channels) {
  if (max_query_len < 2 * kPiece) return 0;
  return (int64_t)num_seqs * ((max_query_len + kPiece - 1) / kPiece) * 2 * channels;
}

extern "C" int vla_seq_mingru_scan(void* out, int64_t out_stride, const void* zp, int64_t z_stride,
                                   const void* up, int64_t u_stride, const void* gp,
                                   int64_t g_stride, float* state, const int* query_start_loc,
                                   const int* context_lens, const int* state_slots, int num_seqs,
                                   int num_slots, int max_query_len, int channels, float* scratch,
                                   int64_t scratch_floats, int dtype, void* stream) {
  if (num_seqs == 0) return VLA_OK;
  if (!out || !zp || !up || !gp || !state || !query_start_loc || !context_lens || !state_slots ||
      num_seqs < 0 || num_seqs > 65535 || num_slots <= 0 || channels <= 0 || max_query_len < 0 ||
      out_stride < channels || z_stride < channels || u_stride < channels || g_stride < channels)
    return VLA_ERR_ARG;
  return with_dtype(dtype, [&](auto s) {
    using S = decltype(s);
    using T = typename S::T;
    const MinGRUGate<S> r{(const T*)zp, z_stride, (const T*)up, u_stride, (const T*)gp, g_stride,
                          (T*)out, out_stride};
    return run_gated_scan(r, state, query_start_loc, context_lens, state_slots, num_seqs,
                          max_query_len, channels, scratch, scratch_floats, (hipStream_t)stream);
  });
}

extern "C" int vla_seq_rglru_scan(void* out, int64_t out_stride, int out_dtype, const float* rp,
                                  int64_t r_stride, const float* ip, int64_t i_stride,
                                  int gate_block, int64_t gate_block_stride,
                                  const float* up, int64_t u_stride, const float* yp,
                                  int64_t y_stride, const float* rate, float* state,
                                  const int* query_start_loc, const int* context_lens,
                                  const int* state_slots, int num_seqs, int num_slots,
                                  int max_query_len, int channels, float* scratch,
                                  int64_t scratch_floats, void* stream) {
  if (num_seqs == 0) return VLA_OK;
  if (!out || !rp || !ip || !up || !yp || !rate || !state || !query_start_loc || !context_lens ||
      !state_slots || num_seqs < 0 || num_seqs > 65535 || num_slots <= 0 || channels <= 0 ||
      max_query_len < 0 || out_stride < channels || gate_block <= 0 || channels % gate_block != 0 ||
      gate_block_stride < 0 || u_stride < channels || y_stride < channels)
    return VLA_ERR_ARG;
  return with_dtype(out_dtype, [&](auto s) {
    using S = decltype(s);
    const RGLRUGate<S> r{rp, r_stride, ip, i_stride, up, u_stride, yp, y_stride, rate,
                         (typename S::T*)out, out_stride, gate_block, gate_block_stride};
    return run_gated_scan(r, state, query_start_loc, context_lens, state_slots, num_seqs,
                          max_query_len, channels, scratch, scratch_floats, (hipStream_t)stream);
  });
}
