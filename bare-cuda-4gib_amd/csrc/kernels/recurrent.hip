// Mixers that carry per-request state of fixed size from step to step: a causal convolution over time on each
// channel (its last taps - 1 inputs are the state) and the real-gated linear recurrent unit (a float state per
// channel).  A step's rows are grouped by request (seq_start), every request has a state slot (seq_slots); a
// request's state is zero when it is admitted, which is what "zeros before the sequence" means for the convolution
// and "from zero" for the recurrence.  One instantiation per storage type; all arithmetic in float.
#include <math.h>

#include "api.h"
#include "common.h"
#include "mfma.h"

namespace bc4g {
namespace {

constexpr int kBlock = 256;

int grid_for(long total) {
  const long g = (total + kBlock - 1) / kBlock;
  return static_cast<int>(g < 1 ? 1 : (g > 65535 ? 65535 : g));
}

// The input of row `at` of a request, as it is kept: with the input's bias added and rounded to the storage type
// (what the state holds of earlier steps is rounded so too: the result does not depend on where a prompt was cut).
template <typename T>
__device__ inline float conv_input(const T* in, const float* in_bias, long at, int c, long in_row) {
  const float v = to_float(in[at * in_row + c]);
  return in_bias ? to_float(from_float<T>(v + in_bias[c])) : v;
}

// out[t, c] = (add_input ? in[t, c] : 0) + out_bias[c] + sum_j w[j, c] * input(t - taps + 1 + j)[c]   (w: [taps][channels])
template <typename T>
__global__ void causal_conv_kernel(const T* __restrict__ in, const float* __restrict__ in_bias,
                                   const float* __restrict__ w, const float* __restrict__ out_bias, int add_input,
                                   T* __restrict__ out, T* state, const int32_t* __restrict__ row_seq,
                                   const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_slots,
                                   long total, int channels, int taps, long in_row, int single_rows) {
  const long stride = static_cast<long>(blockDim.x) * gridDim.x;
  for (long idx = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; idx < total; idx += stride) {
    const int c = static_cast<int>(idx % channels);
    const long t = idx / channels;
    const int s = row_seq[t];
    const long start = seq_start[s];
    const int local = static_cast<int>(t - start);
    T* tail = state + static_cast<long>(seq_slots[s]) * (taps - 1) * channels;
    float acc = out_bias ? out_bias[c] : 0.f;
    for (int j = 0; j < taps; ++j) {
      const int src = local - (taps - 1) + j;
      const float v = src >= 0 ? conv_input(in, in_bias, start + src, c, in_row)
                               : to_float(tail[static_cast<long>(taps - 1 + src) * channels + c]);
      acc = fmaf(w[static_cast<long>(j) * channels + c], v, acc);
    }
    if (add_input) acc += to_float(in[t * in_row + c]);
    out[idx] = from_float<T>(acc);
    if (single_rows) {      // every request brings one row: this thread alone touches the tail of (request, channel)
      for (int i = 0; i + 1 < taps - 1; ++i) tail[static_cast<long>(i) * channels + c] = tail[static_cast<long>(i + 1) * channels + c];
      if (taps > 1) tail[static_cast<long>(taps - 2) * channels + c] = from_float<T>(conv_input(in, in_bias, t, c, in_row));
    }
  }
}

// The same for bfloat16 and channels in whole pieces of 16 bytes: a thread takes eight channels of one row, the index
// arithmetic once for the eight.
__device__ inline void widen8(const uint4 v, float (&f)[8]) {
  const unsigned w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int e = 0; e < 4; ++e) f[2 * e] = __uint_as_float(w[e] << 16), f[2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u);
}

__global__ void causal_conv_pieces_kernel(const bf16_t* __restrict__ in, const float* __restrict__ in_bias,
                                          const float* __restrict__ w, const float* __restrict__ out_bias, int add_input,
                                          bf16_t* __restrict__ out, bf16_t* state,
                                          const int32_t* __restrict__ row_seq, const int32_t* __restrict__ seq_start,
                                          const int32_t* __restrict__ seq_slots, long total, int channels, int taps, long in_row,
                                          int single_rows) {
  const int pieces = channels / 8;
  const long stride = static_cast<long>(blockDim.x) * gridDim.x;
  for (long idx = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; idx < total; idx += stride) {
    const int c0 = static_cast<int>(idx % pieces) * 8;
    const long t = idx / pieces;
    const int s = row_seq[t];
    const long start = seq_start[s];
    const int local = static_cast<int>(t - start);
    bf16_t* tail = state + static_cast<long>(seq_slots[s]) * (taps - 1) * channels;
    float acc[8], bias[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = out_bias ? out_bias[c0 + e] : 0.f, bias[e] = in_bias ? in_bias[c0 + e] : 0.f;
    for (int j = 0; j < taps; ++j) {
      const int src = local - (taps - 1) + j;
      float v[8];
      if (src >= 0) {
        widen8(load16(in + (start + src) * in_row + c0), v);
        if (in_bias) {
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] = to_float(from_float<bf16_t>(v[e] + bias[e]));      // as the tail keeps it
        }
      } else {
        widen8(load16(tail + static_cast<long>(taps - 1 + src) * channels + c0), v);
      }
      const float4 wa = *reinterpret_cast<const float4*>(w + static_cast<long>(j) * channels + c0);
      const float4 wb = *reinterpret_cast<const float4*>(w + static_cast<long>(j) * channels + c0 + 4);
      const float wj[8] = {wa.x, wa.y, wa.z, wa.w, wb.x, wb.y, wb.z, wb.w};
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = fmaf(wj[e], v[e], acc[e]);
    }
    if (add_input) {
      float v[8];
      widen8(load16(in + t * in_row + c0), v);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += v[e];
    }
    unsigned o[4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
      o[e] = static_cast<unsigned>(bf16_bits_from_float(acc[2 * e])) | (static_cast<unsigned>(bf16_bits_from_float(acc[2 * e + 1])) << 16);
    *reinterpret_cast<uint4*>(out + t * channels + c0) = make_uint4(o[0], o[1], o[2], o[3]);
    if (single_rows) {      // every request brings one row: this thread alone touches the tail of (request, these channels)
      for (int i = 0; i + 1 < taps - 1; ++i)
        *reinterpret_cast<uint4*>(tail + static_cast<long>(i) * channels + c0) = load16(tail + static_cast<long>(i + 1) * channels + c0);
      if (taps > 1) {
        float v[8];
        widen8(load16(in + t * in_row + c0), v);
        unsigned k[4];
#pragma unroll
        for (int e = 0; e < 4; ++e)
          k[e] = static_cast<unsigned>(bf16_bits_from_float(v[2 * e] + bias[2 * e])) |
                 (static_cast<unsigned>(bf16_bits_from_float(v[2 * e + 1] + bias[2 * e + 1])) << 16);
        *reinterpret_cast<uint4*>(tail + static_cast<long>(taps - 2) * channels + c0) = make_uint4(k[0], k[1], k[2], k[3]);
      }
    }
  }
}

// The state after the step: the last taps - 1 inputs of (what the state held, then the step's rows).  A thread takes one
// (request, channel) and walks the taps in ascending order: what it reads lies behind what it has written.
template <typename T>
__global__ void causal_conv_state_kernel(const T* __restrict__ in, const float* __restrict__ in_bias, T* __restrict__ state,
                                         const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_slots,
                                         long total, int channels, int taps, long in_row) {
  const long stride = static_cast<long>(blockDim.x) * gridDim.x;
  for (long idx = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; idx < total; idx += stride) {
    const int c = static_cast<int>(idx % channels);
    const int s = static_cast<int>(idx / channels);
    const long start = seq_start[s];
    const int n = static_cast<int>(seq_start[s + 1] - start);
    T* tail = state + static_cast<long>(seq_slots[s]) * (taps - 1) * channels;
    for (int i = 0; i < taps - 1; ++i) {
      const int src = n - (taps - 1) + i;
      tail[static_cast<long>(i) * channels + c] =
          src >= 0 ? from_float<T>(conv_input(in, in_bias, start + src, c, in_row))
                   : tail[static_cast<long>(i + n) * channels + c];
    }
  }
}

__device__ inline float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ inline float softplus_f(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }
__device__ inline float gelu_tanh_f(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

constexpr int kChunk = 64;         // rows of a request that one thread walks

// Decay and drive of one row and channel from the gates' sums: r = sigmoid(sum_a + ba), i = sigmoid(sum_i + bi),
// a = exp(-8 r softplus(lam)), drive = sqrt(1 - a^2) i u  (1 - a^2 as -expm1(2 log a): exact also where a is close to 1).
__device__ inline void decay_and_drive(float sum_a, float sum_i, float u, float ba, float bi, float sp, float* a, float* x) {
  const float log_a = -8.0f * sigmoid_f(sum_a + ba) * sp;
  *a = expf(log_a);
  *x = sqrtf(-expm1f(2.0f * log_a)) * sigmoid_f(sum_i + bi) * u;
}

// The recurrence S_t = a_t S_(t-1) + x_t over a request's rows in chunks of kChunk, so that a long prompt's rows are
// walked by many threads: a thread takes (channel, chunk, request).  First pass: what the chunk does to a state,
// S_out = A S_in + B; the first chunk's thread also notes the request's state before the step.  Second pass: the
// state before the chunk from the chunks before it, then the chunk's rows for good: out[t] = S_t gelu_tanh(y[t] + by);
// the last chunk's thread leaves the state.  pre [T, blocks, 2 bs] holds the gates' sums (Ra u, then Ri u, of a block).
template <typename T, bool kSecond>
__global__ __launch_bounds__(kWave) void rglru_chunks_kernel(
    const float* __restrict__ pre, const T* __restrict__ u, const T* __restrict__ y, const float* __restrict__ ra_b,
    const float* __restrict__ ri_b, const float* __restrict__ lam, const float* __restrict__ y_bias, T* __restrict__ out,
    float* __restrict__ state, float* __restrict__ chunk_a, float* __restrict__ chunk_b, float* __restrict__ before,
    const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_slots, int width, int bs, int most_chunks,
    long y_row) {
  const int ch = blockIdx.x * kWave + threadIdx.x, chunk = blockIdx.y, s = blockIdx.z;
  const long start = seq_start[s], end = seq_start[s + 1];
  const long lo = start + static_cast<long>(chunk) * kChunk, hi = lo + kChunk < end ? lo + kChunk : end;
  if (ch >= width || lo >= end) return;
  const int b = ch / bs, o = ch - b * bs;
  const float ba = ra_b[ch], bi = ri_b[ch], sp = softplus_f(lam[ch]);
  const float* pa = pre + static_cast<long>(b) * 2 * bs + o;           // + t * 2 * width; the other gate bs further
  float* slot = state + static_cast<long>(seq_slots[s]) * width + ch;
  const long note = (static_cast<long>(s) * most_chunks) * width + ch;   // + chunk * width
  if (!kSecond) {
    float A = 1.f, B = 0.f;
    for (long t = lo; t < hi; ++t) {
      float a, x;
      decay_and_drive(pa[t * 2 * width], pa[t * 2 * width + bs], to_float(u[t * width + ch]), ba, bi, sp, &a, &x);
      B = fmaf(a, B, x);
      A *= a;
    }
    chunk_a[note + static_cast<long>(chunk) * width] = A;
    chunk_b[note + static_cast<long>(chunk) * width] = B;
    if (chunk == 0) before[static_cast<long>(s) * width + ch] = *slot;
  } else {
    float st = before[static_cast<long>(s) * width + ch];
    for (int c = 0; c < chunk; ++c) st = fmaf(chunk_a[note + static_cast<long>(c) * width], st, chunk_b[note + static_cast<long>(c) * width]);
    const float yb = y_bias ? y_bias[ch] : 0.f;
    for (long t = lo; t < hi; ++t) {
      float a, x;
      decay_and_drive(pa[t * 2 * width], pa[t * 2 * width + bs], to_float(u[t * width + ch]), ba, bi, sp, &a, &x);
      st = fmaf(a, st, x);
      out[t * width + ch] = from_float<T>(st * gelu_tanh_f(to_float(y[t * y_row + ch]) + yb));
    }
    if (hi == end) *slot = st;
  }
}

}  // namespace
}  // namespace bc4g

using namespace bc4g;

extern "C" int bc4g_causal_conv(const void* in, int dtype, const float* in_bias, const float* w, const float* out_bias,
                                int add_input, void* out, void* state, const int32_t* row_seq, const int32_t* seq_start,
                                const int32_t* seq_slots, int n_rows, int n_seqs, int channels, int taps, long in_row,
                                void* stream) {
  BC4G_REQUIRE(n_rows >= 0 && n_seqs >= 0 && channels > 0 && taps >= 1, "causal_conv: bad sizes T=%d S=%d C=%d taps=%d",
               n_rows, n_seqs, channels, taps);
  BC4G_REQUIRE(in && w && out && in != out && row_seq && seq_start && seq_slots && (taps == 1 || state) && in_row >= channels,
               "causal_conv: a tensor is missing (or the output is the input, or the input's rows are shorter than the channels)");
  if (n_rows == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const long total = static_cast<long>(n_rows) * channels, per_seq = static_cast<long>(n_seqs) * channels;
  // every request brings one row (a decode step): the thread that computes a row's channel also moves its tail
  const int single_rows = n_rows == n_seqs ? 1 : 0;
#define BC4G_CONV(T)                                                                                                      \
  do {                                                                                                                    \
    causal_conv_kernel<T><<<grid_for(total), kBlock, 0, s>>>(static_cast<const T*>(in), in_bias, w, out_bias, add_input, \
                                                             static_cast<T*>(out), static_cast<T*>(state), row_seq,       \
                                                             seq_start, seq_slots, total, channels, taps, in_row,         \
                                                             single_rows);                                                \
    if (taps > 1 && !single_rows)                                                                                         \
      causal_conv_state_kernel<T><<<grid_for(per_seq), kBlock, 0, s>>>(static_cast<const T*>(in), in_bias,                \
                                                                       static_cast<T*>(state), seq_start, seq_slots,      \
                                                                       per_seq, channels, taps, in_row);                  \
  } while (0)
  const bool pieces = dtype == kBF16 && channels % 8 == 0 && in_row % 8 == 0 && reinterpret_cast<uintptr_t>(in) % 16 == 0 &&
                      reinterpret_cast<uintptr_t>(w) % 16 == 0 &&
                      reinterpret_cast<uintptr_t>(out) % 16 == 0 && (taps == 1 || reinterpret_cast<uintptr_t>(state) % 16 == 0);
  if (dtype == kF32) BC4G_CONV(float);
  else if (pieces) {
    causal_conv_pieces_kernel<<<grid_for(total / 8), kBlock, 0, s>>>(
        static_cast<const bf16_t*>(in), in_bias, w, out_bias, add_input, static_cast<bf16_t*>(out), static_cast<bf16_t*>(state),
        row_seq, seq_start, seq_slots, total / 8, channels, taps, in_row, single_rows);
    if (taps > 1 && !single_rows)
      causal_conv_state_kernel<bf16_t><<<grid_for(per_seq), kBlock, 0, s>>>(static_cast<const bf16_t*>(in), in_bias,
                                                                            static_cast<bf16_t*>(state), seq_start, seq_slots,
                                                                            per_seq, channels, taps, in_row);
  } else if (dtype == kBF16) BC4G_CONV(bf16_t);
  else return fail("causal_conv: unknown dtype %d", dtype);
#undef BC4G_CONV
  return check_launch("causal_conv");
}

extern "C" int bc4g_rglru_scan(const float* pre, const void* u, const void* y, int dtype, const float* ra_b, const float* ri_b,
                               const float* lam, const float* y_bias, void* out, float* state, float* chunk_a, float* chunk_b,
                               float* before, const int32_t* seq_start, const int32_t* seq_slots, int n_rows, int n_seqs,
                               int most_rows, int width, int blocks, long y_row, void* stream) {
  BC4G_REQUIRE(n_rows >= 0 && n_seqs >= 0 && width > 0 && blocks > 0 && width % blocks == 0 && n_seqs <= 65535 && most_rows >= 0,
               "rglru_scan: bad sizes T=%d S=%d W=%d blocks=%d", n_rows, n_seqs, width, blocks);
  BC4G_REQUIRE(pre && u && y && ra_b && ri_b && lam && out && state && chunk_a && chunk_b && before && seq_start && seq_slots &&
               y_row >= width, "rglru_scan: a tensor is missing (or y's rows are shorter than the width)");
  if (n_rows == 0 || n_seqs == 0 || most_rows == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int most_chunks = ceil_div(most_rows, kChunk);
  BC4G_REQUIRE(most_chunks <= 65535, "rglru_scan: %d rows of one request are beyond the grid limit", most_rows);
  dim3 grid(ceil_div(width, kWave), most_chunks, n_seqs);
#define BC4G_SCAN(T)                                                                                                            \
  do {                                                                                                                          \
    rglru_chunks_kernel<T, false><<<grid, kWave, 0, s>>>(pre, static_cast<const T*>(u), static_cast<const T*>(y), ra_b, ri_b,  \
                                                         lam, y_bias, static_cast<T*>(out), state, chunk_a, chunk_b, before,   \
                                                         seq_start, seq_slots, width, width / blocks, most_chunks, y_row);     \
    rglru_chunks_kernel<T, true><<<grid, kWave, 0, s>>>(pre, static_cast<const T*>(u), static_cast<const T*>(y), ra_b, ri_b,   \
                                                        lam, y_bias, static_cast<T*>(out), state, chunk_a, chunk_b, before,    \
                                                        seq_start, seq_slots, width, width / blocks, most_chunks, y_row);      \
  } while (0)
  if (dtype == kF32) BC4G_SCAN(float);
  else if (dtype == kBF16) BC4G_SCAN(bf16_t);
  else return fail("rglru_scan: unknown dtype %d", dtype);
#undef BC4G_SCAN
  return check_launch("rglru_scan");
}
