// Mixers that carry per-request state of fixed size from step to step: a causal convolution over time on each
// channel (its last taps - 1 inputs are the state) and the real-gated linear recurrent unit (a float state per
// channel).  A step's rows are grouped by request (seq_start), every request has a state slot (seq_slots); a
// request's state is zero when it is admitted, which is what "zeros before the sequence" means for the convolution
// and "from zero" for the recurrence.  One instantiation per storage type; all arithmetic in float.
#include <math.h>

#include "api.h"
#include "common.h"

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
__device__ inline float conv_input(const T* in, const float* in_bias, long at, int c, int channels) {
  const float v = to_float(in[at * channels + c]);
  return in_bias ? to_float(from_float<T>(v + in_bias[c])) : v;
}

// out[t, c] = (add_input ? in[t, c] : 0) + out_bias[c] + sum_j w[c, j] * input(t - taps + 1 + j)[c]
template <typename T>
__global__ void causal_conv_kernel(const T* __restrict__ in, const float* __restrict__ in_bias,
                                   const float* __restrict__ w, const float* __restrict__ out_bias, int add_input,
                                   T* __restrict__ out, const T* __restrict__ state, const int32_t* __restrict__ row_seq,
                                   const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_slots,
                                   long total, int channels, int taps) {
  const long stride = static_cast<long>(blockDim.x) * gridDim.x;
  for (long idx = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; idx < total; idx += stride) {
    const int c = static_cast<int>(idx % channels);
    const long t = idx / channels;
    const int s = row_seq[t];
    const long start = seq_start[s];
    const int local = static_cast<int>(t - start);
    const T* tail = state + static_cast<long>(seq_slots[s]) * (taps - 1) * channels;
    float acc = out_bias ? out_bias[c] : 0.f;
    for (int j = 0; j < taps; ++j) {
      const int src = local - (taps - 1) + j;
      const float v = src >= 0 ? conv_input(in, in_bias, start + src, c, channels)
                               : to_float(tail[static_cast<long>(taps - 1 + src) * channels + c]);
      acc = fmaf(w[static_cast<long>(c) * taps + j], v, acc);
    }
    if (add_input) acc += to_float(in[idx]);
    out[idx] = from_float<T>(acc);
  }
}

// The state after the step: the last taps - 1 inputs of (what the state held, then the step's rows).  A thread takes one
// (request, channel) and walks the taps in ascending order: what it reads lies behind what it has written.
template <typename T>
__global__ void causal_conv_state_kernel(const T* __restrict__ in, const float* __restrict__ in_bias, T* __restrict__ state,
                                         const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_slots,
                                         long total, int channels, int taps) {
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
          src >= 0 ? from_float<T>(conv_input(in, in_bias, start + src, c, channels))
                   : tail[static_cast<long>(i + n) * channels + c];
    }
  }
}

__device__ inline float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ inline float softplus_f(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }
__device__ inline float gelu_tanh_f(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

constexpr int kGateRows = 16;      // rows of a workgroup: four a wave
constexpr int kGateChunk = 64;     // inputs staged in LDS at a time

// The gates of the recurrence, for channel ch of block b = ch / bs:  r = sigmoid(Ra[b] u_b + ra_b), i = sigmoid(Ri[b] u_b
// + ri_b); decay[t, ch] = a = exp(-8 r softplus(lam)); drive[t, ch] = sqrt(1 - a^2) i u.  The block matrices come
// transposed, [block][in][out], so that a wave's lanes (one output each) read side by side.  Sums over the inputs
// in ascending order in one thread.
template <typename T, typename TW>
__global__ __launch_bounds__(kBlock) void rglru_gates_kernel(const T* __restrict__ u, const TW* __restrict__ ra_t,
                                                             const TW* __restrict__ ri_t, const float* __restrict__ ra_b,
                                                             const float* __restrict__ ri_b, const float* __restrict__ lam,
                                                             float* __restrict__ decay, float* __restrict__ drive,
                                                             int n_rows, int width, int bs) {
  __shared__ float u_s[kGateRows][kGateChunk];
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int row0 = blockIdx.x * kGateRows, b = blockIdx.y, o = blockIdx.z * kWave + lane;
  const TW* wa = ra_t + static_cast<long>(b) * bs * bs;
  const TW* wi = ri_t + static_cast<long>(b) * bs * bs;
  float sa[4] = {0.f, 0.f, 0.f, 0.f}, si[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < bs; k0 += kGateChunk) {
    const int kn = min(kGateChunk, bs - k0);
    for (int e = threadIdx.x; e < kGateRows * kGateChunk; e += kBlock) {
      const int r = e / kGateChunk, k = e % kGateChunk;
      const int row = row0 + r;
      u_s[r][k] = (row < n_rows && k < kn) ? to_float(u[static_cast<long>(row) * width + b * bs + k0 + k]) : 0.f;
    }
    __syncthreads();
    if (o < bs) {
      for (int k = 0; k < kn; ++k) {
        const float a = to_float(wa[static_cast<long>(k0 + k) * bs + o]), i = to_float(wi[static_cast<long>(k0 + k) * bs + o]);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float uv = u_s[wave * 4 + r][k];
          sa[r] = fmaf(a, uv, sa[r]);
          si[r] = fmaf(i, uv, si[r]);
        }
      }
    }
    __syncthreads();
  }
  if (o >= bs) return;
  const int ch = b * bs + o;
  const float sp = softplus_f(lam[ch]), ba = ra_b[ch], bi = ri_b[ch];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int row = row0 + wave * 4 + r;
    if (row >= n_rows) continue;
    const float gate_r = sigmoid_f(sa[r] + ba), gate_i = sigmoid_f(si[r] + bi);
    const float log_a = -8.0f * gate_r * sp;
    const long at = static_cast<long>(row) * width + ch;
    decay[at] = expf(log_a);
    drive[at] = sqrtf(-expm1f(2.0f * log_a)) * gate_i * to_float(u[at]);
  }
}

// S_t = decay_t S_(t-1) + drive_t along a request's rows, from the request's state and back into it;
// out[t] = S_t * gelu_tanh(y[t] + y_bias).  A thread takes one (request, channel).
template <typename T>
__global__ void rglru_scan_kernel(const float* __restrict__ decay, const float* __restrict__ drive, const T* __restrict__ y,
                                  const float* __restrict__ y_bias, T* __restrict__ out, float* __restrict__ state,
                                  const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_slots, int width) {
  const int ch = blockIdx.x * blockDim.x + threadIdx.x, s = blockIdx.y;
  if (ch >= width) return;
  const long start = seq_start[s], end = seq_start[s + 1];
  float* slot = state + static_cast<long>(seq_slots[s]) * width + ch;
  const float yb = y_bias ? y_bias[ch] : 0.f;
  float st = *slot;
  for (long t = start; t < end; ++t) {
    const long at = t * width + ch;
    st = fmaf(decay[at], st, drive[at]);
    out[at] = from_float<T>(st * gelu_tanh_f(to_float(y[at]) + yb));
  }
  *slot = st;
}

}  // namespace
}  // namespace bc4g

using namespace bc4g;

extern "C" int bc4g_causal_conv(const void* in, int dtype, const float* in_bias, const float* w, const float* out_bias,
                                int add_input, void* out, void* state, const int32_t* row_seq, const int32_t* seq_start,
                                const int32_t* seq_slots, int n_rows, int n_seqs, int channels, int taps, void* stream) {
  BC4G_REQUIRE(n_rows >= 0 && n_seqs >= 0 && channels > 0 && taps >= 1, "causal_conv: bad sizes T=%d S=%d C=%d taps=%d",
               n_rows, n_seqs, channels, taps);
  BC4G_REQUIRE(in && w && out && in != out && row_seq && seq_start && seq_slots && (taps == 1 || state),
               "causal_conv: a tensor is missing (or the output is the input)");
  if (n_rows == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const long total = static_cast<long>(n_rows) * channels, per_seq = static_cast<long>(n_seqs) * channels;
#define BC4G_CONV(T)                                                                                                      \
  do {                                                                                                                    \
    causal_conv_kernel<T><<<grid_for(total), kBlock, 0, s>>>(static_cast<const T*>(in), in_bias, w, out_bias, add_input, \
                                                             static_cast<T*>(out), static_cast<const T*>(state), row_seq, \
                                                             seq_start, seq_slots, total, channels, taps);                \
    if (taps > 1)                                                                                                         \
      causal_conv_state_kernel<T><<<grid_for(per_seq), kBlock, 0, s>>>(static_cast<const T*>(in), in_bias,                \
                                                                       static_cast<T*>(state), seq_start, seq_slots,      \
                                                                       per_seq, channels, taps);                          \
  } while (0)
  if (dtype == kF32) BC4G_CONV(float);
  else if (dtype == kBF16) BC4G_CONV(bf16_t);
  else return fail("causal_conv: unknown dtype %d", dtype);
#undef BC4G_CONV
  return check_launch("causal_conv");
}

extern "C" int bc4g_rglru_gates(const void* u, int dtype, const void* ra_t, const void* ri_t, int w_dtype, const float* ra_b,
                                const float* ri_b, const float* lam, float* decay, float* drive, int n_rows, int width,
                                int blocks, void* stream) {
  BC4G_REQUIRE(n_rows >= 0 && width > 0 && blocks > 0 && width % blocks == 0, "rglru_gates: bad sizes T=%d W=%d blocks=%d",
               n_rows, width, blocks);
  BC4G_REQUIRE(u && ra_t && ri_t && ra_b && ri_b && lam && decay && drive, "rglru_gates: a tensor is missing");
  BC4G_REQUIRE(blocks <= 65535, "rglru_gates: %d blocks are beyond the grid limit", blocks);
  if (n_rows == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int bs = width / blocks;
  dim3 grid(ceil_div(n_rows, kGateRows), blocks, ceil_div(bs, kWave));
#define BC4G_GATES(T, TW)                                                                                            \
  rglru_gates_kernel<T, TW><<<grid, kBlock, 0, s>>>(static_cast<const T*>(u), static_cast<const TW*>(ra_t),         \
                                                    static_cast<const TW*>(ri_t), ra_b, ri_b, lam, decay, drive,    \
                                                    n_rows, width, bs)
  if (dtype == kF32 && w_dtype == kF32) BC4G_GATES(float, float);
  else if (dtype == kBF16 && w_dtype == kBF16) BC4G_GATES(bf16_t, bf16_t);
  else if (dtype == kBF16 && w_dtype == kF32) BC4G_GATES(bf16_t, float);
  else if (dtype == kF32 && w_dtype == kBF16) BC4G_GATES(float, bf16_t);
  else return fail("rglru_gates: unknown dtypes %d, %d", dtype, w_dtype);
#undef BC4G_GATES
  return check_launch("rglru_gates");
}

extern "C" int bc4g_rglru_scan(const float* decay, const float* drive, const void* y, int dtype, const float* y_bias, void* out,
                               float* state, const int32_t* seq_start, const int32_t* seq_slots, int n_rows, int n_seqs,
                               int width, void* stream) {
  BC4G_REQUIRE(n_rows >= 0 && n_seqs >= 0 && width > 0 && n_seqs <= 65535, "rglru_scan: bad sizes T=%d S=%d W=%d", n_rows,
               n_seqs, width);
  BC4G_REQUIRE(decay && drive && y && out && state && seq_start && seq_slots, "rglru_scan: a tensor is missing");
  if (n_rows == 0 || n_seqs == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid(ceil_div(width, kWave), n_seqs);
  if (dtype == kF32)
    rglru_scan_kernel<float><<<grid, kWave, 0, s>>>(decay, drive, static_cast<const float*>(y), y_bias,
                                                    static_cast<float*>(out), state, seq_start, seq_slots, width);
  else if (dtype == kBF16)
    rglru_scan_kernel<bf16_t><<<grid, kWave, 0, s>>>(decay, drive, static_cast<const bf16_t*>(y), y_bias,
                                                     static_cast<bf16_t*>(out), state, seq_start, seq_slots, width);
  else return fail("rglru_scan: unknown dtype %d", dtype);
  return check_launch("rglru_scan");
}
