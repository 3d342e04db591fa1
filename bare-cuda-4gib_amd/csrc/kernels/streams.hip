// A residual stream kept in several copies (hyper-connections), and the Dynamic Tanh norm that reads it.
//
// The copies of a row lie side by side: x [T, n, H] float32.  A sublayer reads one weighted sum of the copies,
//   u = sum_s read[s] x[s],
// and writes all copies at once from the old ones and its output y,
//   x'[t] = sum_s mix[s, t] x[s] + write[t] y        (mix is indexed [from, to]).
// The norm is pointwise -- tanh(alpha u) * g + b, no mean and no variance -- so it rides along with the read, and the
// read of the next sublayer rides along with the write before it (the new copies are in registers then).
// Everything is float32 arithmetic; only what a product reads is stored in the activations' type.
#include <math.h>

#include "api.h"
#include "common.h"

namespace bc4g {
namespace {

constexpr int kBlock = 256;
constexpr int kMaxStreams = 16;

int grid_for(long total) {
  const long g = (total + kBlock - 1) / kBlock;
  return static_cast<int>(g < 1 ? 1 : (g > 1048576 ? 1048576 : g));
}

__device__ inline float dyt(float u, float alpha, float g, float b, float out_scale) {
  return (tanhf(alpha * u) * g + b) * out_scale;
}

// out[r, c] = N(sum_s read[s] x[rows ? rows[r] : r, s, c]);  read null: every copy counts once;  alpha null: no norm.
template <typename TO>
__global__ void streams_read_kernel(const float* __restrict__ x, const int32_t* __restrict__ rows,
                                    const float* __restrict__ read, const float* __restrict__ alpha,
                                    const float* __restrict__ g, const float* __restrict__ b, float out_scale,
                                    TO* __restrict__ out, long total, int n, int hidden) {
  const long stride = static_cast<long>(blockDim.x) * gridDim.x;
  const float a = alpha ? alpha[0] : 0.f;
  for (long idx = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; idx < total; idx += stride) {
    const int c = static_cast<int>(idx % hidden);
    const long r = idx / hidden;
    const long src = rows ? rows[r] : r;
    const float* xr = x + src * n * hidden + c;
    float u = 0.f;
    for (int s = 0; s < n; ++s) u = fmaf(read ? read[s] : 1.0f, xr[static_cast<long>(s) * hidden], u);
    out[idx] = from_float<TO>(alpha ? dyt(u, a, g[c], b[c], out_scale) : u);
  }
}

// The write, and with next_out the next reader's input from the new copies.  NS: the most copies this instance holds in
// registers (4, 8 or 16).
template <typename TO, int NS>
__global__ void streams_write_kernel(float* __restrict__ x, const float* __restrict__ y, const float* __restrict__ mix,
                                     const float* __restrict__ write, const float* __restrict__ next_read,
                                     const float* __restrict__ alpha, const float* __restrict__ g,
                                     const float* __restrict__ b, TO* __restrict__ next_out, long total, int n, int hidden) {
  __shared__ float mix_s[kMaxStreams * kMaxStreams], write_s[kMaxStreams], read_s[kMaxStreams];
  for (int i = threadIdx.x; i < n * n; i += blockDim.x) mix_s[i] = mix[i];
  for (int i = threadIdx.x; i < n; i += blockDim.x) write_s[i] = write[i], read_s[i] = next_read ? next_read[i] : 0.f;
  __syncthreads();
  const long stride = static_cast<long>(blockDim.x) * gridDim.x;
  const float a = alpha ? alpha[0] : 0.f;
  for (long idx = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; idx < total; idx += stride) {
    const int c = static_cast<int>(idx % hidden);
    const long r = idx / hidden;
    float* xr = x + r * n * hidden + c;
    float old[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) old[s] = s < n ? xr[static_cast<long>(s) * hidden] : 0.f;
    const float yv = y[idx];
    float u = 0.f;
#pragma unroll
    for (int t = 0; t < NS; ++t) {
      if (t >= n) break;
      float acc = 0.f;
#pragma unroll
      for (int s = 0; s < NS; ++s)
        if (s < n) acc = fmaf(mix_s[s * n + t], old[s], acc);
      acc = fmaf(write_s[t], yv, acc);
      xr[static_cast<long>(t) * hidden] = acc;
      u = fmaf(read_s[t], acc, u);
    }
    if (next_out) next_out[idx] = from_float<TO>(alpha ? dyt(u, a, g[c], b[c], 1.0f) : u);
  }
}

// The write for rows of whole pieces of four channels (H a multiple of 4, the tensors on 16-byte borders): a thread takes
// four neighbouring channels of one row.  The same sums in the same order as above.
template <typename TO, int NS>
__global__ void streams_write_four_kernel(float* __restrict__ x, const float* __restrict__ y, const float* __restrict__ mix,
                                          const float* __restrict__ write, const float* __restrict__ next_read,
                                          const float* __restrict__ alpha, const float* __restrict__ g,
                                          const float* __restrict__ b, TO* __restrict__ next_out, long total, int n, int hidden) {
  __shared__ float mix_s[kMaxStreams * kMaxStreams], write_s[kMaxStreams], read_s[kMaxStreams];
  for (int i = threadIdx.x; i < n * n; i += blockDim.x) mix_s[i] = mix[i];
  for (int i = threadIdx.x; i < n; i += blockDim.x) write_s[i] = write[i], read_s[i] = next_read ? next_read[i] : 0.f;
  __syncthreads();
  const long stride = static_cast<long>(blockDim.x) * gridDim.x;
  const float a = alpha ? alpha[0] : 0.f;
  const int per_row = hidden / 4;
  for (long idx = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; idx < total; idx += stride) {
    const int c = static_cast<int>(idx % per_row) * 4;
    const long r = idx / per_row;
    float* xr = x + r * n * hidden + c;
    float4 old[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s)
      old[s] = s < n ? *reinterpret_cast<const float4*>(xr + static_cast<long>(s) * hidden) : make_float4(0.f, 0.f, 0.f, 0.f);
    const float4 yv = *reinterpret_cast<const float4*>(y + r * hidden + c);
    float4 u = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int t = 0; t < NS; ++t) {
      if (t >= n) break;
      float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int s = 0; s < NS; ++s)
        if (s < n) {
          const float m = mix_s[s * n + t];
          acc.x = fmaf(m, old[s].x, acc.x), acc.y = fmaf(m, old[s].y, acc.y), acc.z = fmaf(m, old[s].z, acc.z), acc.w = fmaf(m, old[s].w, acc.w);
        }
      const float w = write_s[t], rd = read_s[t];
      acc.x = fmaf(w, yv.x, acc.x), acc.y = fmaf(w, yv.y, acc.y), acc.z = fmaf(w, yv.z, acc.z), acc.w = fmaf(w, yv.w, acc.w);
      *reinterpret_cast<float4*>(xr + static_cast<long>(t) * hidden) = acc;
      u.x = fmaf(rd, acc.x, u.x), u.y = fmaf(rd, acc.y, u.y), u.z = fmaf(rd, acc.z, u.z), u.w = fmaf(rd, acc.w, u.w);
    }
    if (next_out) {
      const float uu[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) next_out[r * hidden + c + i] = from_float<TO>(alpha ? dyt(uu[i], a, g[c + i], b[c + i], 1.0f) : uu[i]);
    }
  }
}

// out[r, s, :] = in[r, :] for every copy s.
__global__ void streams_fill_kernel(const float* __restrict__ in, float* __restrict__ out, long total, int n, int hidden) {
  const long stride = static_cast<long>(blockDim.x) * gridDim.x;
  for (long idx = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; idx < total; idx += stride) {
    const int c = static_cast<int>(idx % hidden);
    const long r = idx / hidden / n;
    out[idx] = in[r * hidden + c];
  }
}

}  // namespace
}  // namespace bc4g

using namespace bc4g;

extern "C" int bc4g_streams_read(const float* x, const int32_t* rows, const float* read, const float* alpha, const float* g,
                                 const float* b, float out_scale, void* out, int out_dtype, int n_rows, int n_streams,
                                 int hidden, void* stream) {
  BC4G_REQUIRE(n_rows >= 0 && n_streams >= 1 && n_streams <= kMaxStreams && hidden > 0,
               "streams_read: bad sizes rows=%d copies=%d (at most %d) H=%d", n_rows, n_streams, kMaxStreams, hidden);
  BC4G_REQUIRE(x && out && (!alpha || (g && b)), "streams_read: a tensor is missing");
  if (n_rows == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const long total = static_cast<long>(n_rows) * hidden;
  if (out_dtype == kF32)
    streams_read_kernel<float><<<grid_for(total), kBlock, 0, s>>>(x, rows, read, alpha, g, b, out_scale,
                                                                  static_cast<float*>(out), total, n_streams, hidden);
  else if (out_dtype == kBF16)
    streams_read_kernel<bf16_t><<<grid_for(total), kBlock, 0, s>>>(x, rows, read, alpha, g, b, out_scale,
                                                                   static_cast<bf16_t*>(out), total, n_streams, hidden);
  else return fail("streams_read: unknown dtype %d", out_dtype);
  return check_launch("streams_read");
}

extern "C" int bc4g_streams_write(float* x, const float* y, const float* mix, const float* write, const float* next_read,
                                  const float* alpha, const float* g, const float* b, void* next_out, int out_dtype,
                                  int n_rows, int n_streams, int hidden, void* stream) {
  BC4G_REQUIRE(n_rows >= 0 && n_streams >= 1 && n_streams <= kMaxStreams && hidden > 0,
               "streams_write: bad sizes rows=%d copies=%d (at most %d) H=%d", n_rows, n_streams, kMaxStreams, hidden);
  BC4G_REQUIRE(x && y && mix && write && (!next_out || next_read) && (!alpha || (g && b)), "streams_write: a tensor is missing");
  if (n_rows == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const long total = static_cast<long>(n_rows) * hidden;
  const bool four = hidden % 4 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0;
#define BC4G_WRITE(TO, NS)                                                                                              \
  do {                                                                                                                  \
    if (four)                                                                                                           \
      streams_write_four_kernel<TO, NS><<<grid_for(total / 4), kBlock, 0, s>>>(x, y, mix, write, next_read, alpha, g, b, \
                                                                               static_cast<TO*>(next_out), total / 4,   \
                                                                               n_streams, hidden);                      \
    else                                                                                                                \
      streams_write_kernel<TO, NS><<<grid_for(total), kBlock, 0, s>>>(x, y, mix, write, next_read, alpha, g, b,          \
                                                                      static_cast<TO*>(next_out), total, n_streams, hidden); \
  } while (0)
#define BC4G_WRITE_N(TO)                                                                                                \
  do { if (n_streams <= 4) BC4G_WRITE(TO, 4); else if (n_streams <= 8) BC4G_WRITE(TO, 8); else BC4G_WRITE(TO, 16); } while (0)
  if (out_dtype == kF32) BC4G_WRITE_N(float);
  else if (out_dtype == kBF16) BC4G_WRITE_N(bf16_t);
  else return fail("streams_write: unknown dtype %d", out_dtype);
#undef BC4G_WRITE_N
#undef BC4G_WRITE
  return check_launch("streams_write");
}

extern "C" int bc4g_streams_fill(const float* in, float* out, int n_rows, int n_streams, int hidden, void* stream) {
  BC4G_REQUIRE(n_rows >= 0 && n_streams >= 1 && hidden > 0 && in && out, "streams_fill: bad arguments rows=%d copies=%d H=%d",
               n_rows, n_streams, hidden);
  if (n_rows == 0) return 0;
  const long total = static_cast<long>(n_rows) * n_streams * hidden;
  streams_fill_kernel<<<grid_for(total), kBlock, 0, static_cast<hipStream_t>(stream)>>>(in, out, total, n_streams, hidden);
  return check_launch("streams_fill");
}
