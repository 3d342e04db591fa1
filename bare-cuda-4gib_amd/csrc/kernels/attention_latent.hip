// Latent attention: every token keeps one low-rank latent (rank numbers, RMS-normed) and one rotated key part (rot
// numbers) that all heads share -- a cache row of rank + rot numbers and nothing per head.  The keys' up-projection
// is absorbed into the query (q_lat[h] = [Wuk[h]^T q_plain[h], rotate(q_rot[h])]), so a score is one dot product of
// rank + rot numbers against the cache row, the weighted sum of the latents is taken per head, and the values'
// up-projection follows on that sum.  The softmax may have a sink per head: a term exp(sink) in the denominator that
// has no key and no value.  Plain float arithmetic, float or bfloat16 cache; rows of prompt portions and single
// decoded tokens are the same to these kernels.
//
//   bc4g_latent_prepare     norms the latent, rotates the shared key part and writes both into the row's cache
//                           slot; rotates every head's rotated query part into the absorbed query
//   bc4g_heads_gemm         out[t, h, :] = w[h] a[t, h, :] for every head (both up-projections)
//   bc4g_attention_latent   the attention itself, over the paged cache
#include <float.h>
#include <math.h>

#include "api.h"
#include "common.h"
#include "mfma.h"

namespace bc4g {
namespace {

constexpr int kPrepBlock = 128;

// Pair i of a rotated vector at position p turns by p * base^(-2 i / dims); the angle in double, so that it is as good
// at position 100,000 as at position 1.
__device__ inline void pair_angle(int pos, int i, int dims, double log_base, float* c, float* s) {
  const double a = static_cast<double>(pos) * exp(-log_base * (2.0 * i) / dims);
  double sd, cd;
  sincos(a, &sd, &cd);
  *c = static_cast<float>(cd);
  *s = static_cast<float>(sd);
}

// The step's table of angles, for every layer with the same rotation to share: table[t][i] = (cos, sin) of pair i at
// the row's position.
__global__ void latent_angles_kernel(const int32_t* __restrict__ positions, float2* __restrict__ table, long total, int half,
                                     double log_base) {
  const long stride = static_cast<long>(blockDim.x) * gridDim.x;
  for (long idx = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; idx < total; idx += stride) {
    float c, s;
    pair_angle(positions[idx / half], static_cast<int>(idx % half), 2 * half, log_base, &c, &s);
    table[idx] = make_float2(c, s);
  }
}

// One workgroup a row.  q: [T, heads, plain + rot] (as projected); dkv: [T, rank + rot] (rows q_row and dkv_row elements
// apart: both may be parts of one product's rows); q_lat: [T, heads, rank + rot]
// float, of which this kernel writes the last rot of every head; the row's cache slot receives [normed latent | rotated
// key part].  Neighbouring elements 2i and 2i + 1 of the first `dims` of a rotated part are a pair; the rest passes.
template <typename T>
__global__ __launch_bounds__(kPrepBlock) void latent_prepare_kernel(
    const T* __restrict__ q, const T* __restrict__ dkv, const float* __restrict__ g, float eps,
    const float* __restrict__ angles, const int32_t* __restrict__ slot_map, T* __restrict__ cache,
    float* __restrict__ q_lat, int heads, int plain, int rot, int rank, int dims, long q_row, long dkv_row) {
  __shared__ float scratch[16];
  extern __shared__ float cs[];                     // [dims / 2][2]: the row's cosines and sines
  const long row = blockIdx.x;
  for (int i = threadIdx.x; i < dims; i += kPrepBlock) cs[i] = angles[row * dims + i];
  // (two workgroups a row: one norms and stores the cache row, the other rotates the queries)
  if (blockIdx.y == 1) {
    __syncthreads();
    const T* qr = q + row * q_row;
    float* ql = q_lat + row * heads * (rank + rot);
    for (int e = threadIdx.x; e < heads * rot; e += kPrepBlock) {
      const int h = e / rot, i = e % rot;
      const T* part = qr + h * (plain + rot) + plain;
      float v = to_float(part[i]);
      if (i < dims) {
        const float c = cs[2 * (i / 2)], s = cs[2 * (i / 2) + 1], other = to_float(part[i ^ 1]);
        v = (i & 1) ? v * c + other * s : v * c - other * s;
      }
      ql[h * (rank + rot) + rank + i] = v;
    }
    return;
  }
  const T* lat = dkv + row * dkv_row;
  float ss = 0.f;
  for (int i = threadIdx.x; i < rank; i += kPrepBlock) {
    const float v = to_float(lat[i]);
    ss += v * v;
  }
  const float scale = 1.0f / sqrtf(block_sum(ss, scratch) / static_cast<float>(rank) + eps);   // (a barrier: cs is written)
  if (cache) {
    T* to = cache + static_cast<long>(slot_map[row]) * (rank + rot);
    for (int i = threadIdx.x; i < rank; i += kPrepBlock) to[i] = from_float<T>(to_float(lat[i]) * scale * g[i]);
    for (int i = threadIdx.x; i < rot; i += kPrepBlock) {
      float v = to_float(lat[rank + i]);
      if (i < dims) {
        const float c = cs[2 * (i / 2)], s = cs[2 * (i / 2) + 1], other = to_float(lat[rank + (i ^ 1)]);
        v = (i & 1) ? v * c + other * s : v * c - other * s;
      }
      to[rank + i] = from_float<T>(v);
    }
  }
}

// ---- a product per head -------------------------------------------------------------------------------------------
// out[t, h, n] = sum_k a[t, h, k] * w[h, n, k]: 64 x 64 outputs a workgroup of 256 threads (4 x 4 a thread), k in steps
// of 16 through LDS, every sum over k in ascending order in one thread.
constexpr int kHT = 64, kHK = 16;

template <typename TA, typename TW, typename TO>
__global__ __launch_bounds__(256) void heads_gemm_kernel(const TA* __restrict__ a, long a_row, long a_head,
                                                         const TW* __restrict__ w, TO* __restrict__ out, long o_row,
                                                         long o_head, int m, int n, int k) {
  __shared__ float a_s[kHK][kHT + 1], w_s[kHK][kHT + 1];
  const int h = blockIdx.z, m0 = blockIdx.x * kHT, n0 = blockIdx.y * kHT;
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  const TA* ah = a + h * a_head;
  const TW* wh = w + static_cast<long>(h) * n * k;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < k; k0 += kHK) {
    for (int e = threadIdx.x; e < kHT * kHK; e += 256) {
      const int r = e / kHK, kk = e % kHK;
      const bool in_k = k0 + kk < k;
      a_s[kk][r] = (in_k && m0 + r < m) ? to_float(ah[(m0 + r) * a_row + k0 + kk]) : 0.f;
      w_s[kk][r] = (in_k && n0 + r < n) ? to_float(wh[static_cast<long>(n0 + r) * k + k0 + kk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kHK; ++kk) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = a_s[kk][ty * 4 + i], wv[i] = w_s[kk][tx * 4 + i];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int r = m0 + ty * 4 + i, c = n0 + tx * 4 + j;
      if (r < m && c < n) out[r * o_row + h * o_head + c] = from_float<TO>(acc[i][j]);
    }
}

// The same on the matrix cores for bfloat16 weights: a wave takes 16 rows x 16 NB columns of one head; both operands
// have k side by side in memory, so a lane's eight k-slots are one load of 16 bytes (activations in float32 are
// rounded to bfloat16 on the way); no LDS.  k a multiple of 8, every row and head of a on a 16-byte boundary.
__device__ inline uint4 load_slots(const bf16_t* p) { return load16(p); }
__device__ inline uint4 load_slots(const float* p) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  auto two = [](float lo, float hi) {
    return static_cast<unsigned>(bf16_bits_from_float(lo)) | (static_cast<unsigned>(bf16_bits_from_float(hi)) << 16);
  };
  return make_uint4(two(a.x, a.y), two(a.z, a.w), two(b.x, b.y), two(b.z, b.w));
}

// KW waves of a workgroup take every KW-th k-step and add their sums up through LDS (few rows: more waves on the
// weights' way in).
template <typename TA, typename TO, int NB, int KW>
__global__ __launch_bounds__(kWave * KW) void heads_mfma_kernel(const TA* __restrict__ a, long a_row, long a_head,
                                                                const bf16_t* __restrict__ w, TO* __restrict__ out, long o_row,
                                                                long o_head, int m, int n, int k) {
  __shared__ floatx4 sums[KW > 1 ? KW : 1][NB][kWave];
  const int h = blockIdx.z, m0 = blockIdx.x * 16, n0 = blockIdx.y * 16 * NB;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int c = lane % 16, g = lane / 16;
  const bool row_there = m0 + c < m;
  const TA* arow = a + (m0 + c) * a_row + h * a_head + 8 * g;
  const bf16_t* wcol[NB];
  bool col_there[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    col_there[nb] = n0 + nb * 16 + c < n;
    wcol[nb] = w + (static_cast<long>(h) * n + n0 + nb * 16 + c) * k + 8 * g;
  }
  floatx4 acc[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) acc[nb] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 8
  for (int k0 = 32 * wave; k0 < k; k0 += 32 * KW) {
    const bool k_there = k0 + 8 * g < k;
    const uint4 av = row_there && k_there ? load_slots(arow + k0) : zero16();
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      const uint4 wv = col_there[nb] && k_there ? load16(wcol[nb] + k0) : zero16();
      acc[nb] = mfma_16x16x32(av, wv, acc[nb]);
    }
  }
  if (KW > 1) {
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) sums[wave][nb][lane] = acc[nb];
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int other = 1; other < KW; ++other) acc[nb] += sums[other][nb][lane];
  }
  // a lane holds column c of every block and rows 4g .. 4g + 3
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    if (!col_there[nb]) continue;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = m0 + 4 * g + i;
      if (r < m) out[r * o_row + h * o_head + n0 + nb * 16 + c] = from_float<TO>(acc[nb][i]);
    }
  }
}

// ---- the attention ---------------------------------------------------------------------------------------------------
// A workgroup takes one row and up to kHeadsPerGroup of its heads, a wave a head: all heads read the same cache rows,
// so a tile of 64 keys goes through LDS once for the group, 64 numbers of every key at a time -- first all of a row for
// the scores (lane = key, the sum over the numbers in ascending order), then, once the tile's weights are known, its
// latent part again for the output (lane = number, the sum over the keys in ascending order).  Keys are walked in
// ascending order from the first the row sees, with a running maximum and sum; the sink joins the sum at the end.
constexpr int kMaxLatentRow = 1024;                   // rank + rot at most
constexpr int kLatentChunks = kMaxLatentRow / kWave;
constexpr int kHeadsPerGroup = 8;
constexpr int kTilePad = kWave + 1;

template <typename T>
__global__ void attention_latent_kernel(const float* __restrict__ q_lat, float* __restrict__ out, const T* __restrict__ cache,
                                        const float* __restrict__ sink, const int32_t* __restrict__ block_table,
                                        int table_stride, const int32_t* __restrict__ row_seq,
                                        const int32_t* __restrict__ positions, int heads, int rank, int row_len,
                                        int page_tokens, int window, float scale) {
  extern __shared__ float lds[];
  const int group = blockDim.x / kWave;
  float* q_s = lds;                                   // [group][row_len]
  float* p_s = q_s + group * row_len;                 // [group][64]
  float* tile = p_s + group * kWave;                  // [64][kTilePad]
  const int row = blockIdx.x, lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int head = blockIdx.y * group + wave;
  const bool live = head < heads;
  const int pos = positions[row];
  const int32_t* table = block_table + static_cast<long>(row_seq[row]) * table_stride;
  if (live) {
    const float* q = q_lat + (static_cast<long>(row) * heads + head) * row_len;
    for (int c = lane; c < row_len; c += kWave) q_s[wave * row_len + c] = q[c];
  }
  __syncthreads();
  const int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  float m = -INFINITY, l = 0.f;
  float acc[kLatentChunks];
#pragma unroll
  for (int i = 0; i < kLatentChunks; ++i) acc[i] = 0.f;

  for (int j0 = first; j0 <= pos; j0 += kWave) {
    const int n_here = min(kWave, pos - j0 + 1);
    const bool seen = j0 + lane <= pos;
    float dot = 0.f;
    for (int c0 = 0; c0 < row_len; c0 += kWave) {
      const int width = min(kWave, row_len - c0);
      // the tile's keys, 64 numbers of each: a wave takes every group-th key, its lanes the key's numbers side by side
      for (int kk = wave; kk < n_here; kk += group) {
        const int jk = j0 + kk;
        const long page = table[jk / page_tokens];
        if (lane < width) tile[kk * kTilePad + lane] = to_float(cache[(page * page_tokens + jk % page_tokens) * row_len + c0 + lane]);
      }
      __syncthreads();
      if (seen && live) {
        const float* qc = q_s + wave * row_len + c0;
        const float* tk = tile + lane * kTilePad;
        for (int c = 0; c < width; ++c) dot = fmaf(qc[c], tk[c], dot);
      }
      __syncthreads();
    }
    const float s = seen ? dot * scale : -INFINITY;
    const float m_new = fmaxf(m, wave_max(s));        // finite: key j0 is always visible
    const float p = seen ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);              // 0 on the first tile (m = -inf)
    l = l * alpha + wave_sum(p);
    m = m_new;
    p_s[wave * kWave + lane] = p;
#pragma unroll
    for (int i = 0; i < kLatentChunks; ++i) acc[i] *= alpha;
#pragma unroll
    for (int i = 0; i < kLatentChunks; ++i) {
      const int c0 = i * kWave;
      if (c0 >= rank) break;
      const int width = min(kWave, rank - c0);
      for (int kk = wave; kk < n_here; kk += group) {
        const int jk = j0 + kk;
        const long page = table[jk / page_tokens];
        if (lane < width) tile[kk * kTilePad + lane] = to_float(cache[(page * page_tokens + jk % page_tokens) * row_len + c0 + lane]);
      }
      __syncthreads();                                // (also: every lane's p is in p_s)
      if (lane < width && live) {
        const float* pw = p_s + wave * kWave;
        for (int jj = 0; jj < n_here; ++jj) acc[i] = fmaf(pw[jj], tile[jj * kTilePad + lane], acc[i]);
      }
      __syncthreads();
    }
  }
  if (!live) return;
  if (sink) l += expf(sink[head] - m);
  const float inv_l = 1.0f / l;
  float* o = out + (static_cast<long>(row) * heads + head) * rank;
#pragma unroll
  for (int i = 0; i < kLatentChunks; ++i) {
    const int c = lane + i * kWave;
    if (c < rank) o[c] = acc[i] * inv_l;
  }
}

}  // namespace
}  // namespace bc4g

using namespace bc4g;

extern "C" int bc4g_latent_angles(const int32_t* positions, float* table, int n_rows, int dims, float base, void* stream) {
  BC4G_REQUIRE(n_rows >= 0 && dims > 0 && dims % 2 == 0 && base > 0.f && positions && table,
               "latent_angles: bad arguments (T=%d, %d rotated dimensions, base %g)", n_rows, dims, base);
  if (n_rows == 0) return 0;
  const long total = static_cast<long>(n_rows) * (dims / 2);
  const long blocks = (total + 255) / 256;
  latent_angles_kernel<<<static_cast<unsigned>(blocks > 65535 ? 65535 : blocks), 256, 0, static_cast<hipStream_t>(stream)>>>(
      positions, reinterpret_cast<float2*>(table), total, dims / 2, log(static_cast<double>(base)));
  return check_launch("latent_angles");
}

extern "C" int bc4g_latent_prepare(const void* q, const void* dkv, int dtype, const float* g, float eps,
                                   const float* angles, const int32_t* slot_map, void* cache, float* q_lat,
                                   int n_rows, int heads, int plain, int rot, int rank, int dims, long q_row, long dkv_row,
                                   void* stream) {
  BC4G_REQUIRE(n_rows >= 0 && heads > 0 && plain >= 0 && rot >= 0 && rank > 0, "latent_prepare: bad sizes T=%d heads=%d "
               "plain=%d rot=%d rank=%d", n_rows, heads, plain, rot, rank);
  BC4G_REQUIRE(dims >= 0 && dims % 2 == 0 && dims <= rot && dims <= 8192,
               "latent_prepare: %d rotated dimensions of %d (even, at most the rotated part)", dims, rot);
  BC4G_REQUIRE(q && dkv && g && (angles || dims == 0) && q_lat && (!cache || slot_map), "latent_prepare: a tensor is missing");
  BC4G_REQUIRE(q_row >= static_cast<long>(heads) * (plain + rot) && dkv_row >= rank + rot, "latent_prepare: rows shorter than their parts");
  if (n_rows == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const size_t lds = static_cast<size_t>(dims > 0 ? dims : 2) * sizeof(float);
  if (dtype == kF32)
    latent_prepare_kernel<float><<<dim3(n_rows, 2), kPrepBlock, lds, s>>>(static_cast<const float*>(q), static_cast<const float*>(dkv), g,
                                                                 eps, angles, slot_map, static_cast<float*>(cache), q_lat,
                                                                 heads, plain, rot, rank, dims, q_row, dkv_row);
  else if (dtype == kBF16)
    latent_prepare_kernel<bf16_t><<<dim3(n_rows, 2), kPrepBlock, lds, s>>>(static_cast<const bf16_t*>(q), static_cast<const bf16_t*>(dkv),
                                                                  g, eps, angles, slot_map, static_cast<bf16_t*>(cache),
                                                                  q_lat, heads, plain, rot, rank, dims, q_row, dkv_row);
  else return fail("latent_prepare: unknown dtype %d", dtype);
  return check_launch("latent_prepare");
}

extern "C" int bc4g_heads_gemm(const void* a, int a_dtype, long a_row, long a_head, const void* w, int w_dtype, void* out,
                               int out_dtype, long o_row, long o_head, int m, int n, int k, int heads, void* stream) {
  BC4G_REQUIRE(m >= 0 && n > 0 && k > 0 && heads > 0 && heads <= 65535, "heads_gemm: bad sizes m=%d n=%d k=%d heads=%d", m, n, k, heads);
  BC4G_REQUIRE(a && w && out && a_row >= k && o_row >= n && a_head >= 0 && o_head >= 0, "heads_gemm: bad operands or strides");
  BC4G_REQUIRE(ceil_div(n, kHT) <= 65535, "heads_gemm: n=%d is beyond the grid limit", n);
  if (m == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // bfloat16 weights with k in whole pieces of 16 bytes: the matrix cores
  const int a_bytes = a_dtype == kBF16 ? 2 : 4;
  if (w_dtype == kBF16 && k % 8 == 0 && a_row % 8 == 0 && a_head % 8 == 0 && reinterpret_cast<uintptr_t>(a) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(w) % 16 == 0 && (a_bytes == 2 || a_dtype == kF32) && (out_dtype == kF32 || out_dtype == kBF16)) {
    // few rows (a decode step): a wave takes one block of 16 columns, so that more waves share the weights' way in
    const int nb = m <= 32 ? 1 : 4;
    dim3 mgrid(ceil_div(m, 16), ceil_div(n, 16 * nb), heads);
    BC4G_REQUIRE(mgrid.y <= 65535, "heads_gemm: n=%d is beyond the grid limit", n);
    const bf16_t* wp = static_cast<const bf16_t*>(w);
#define BC4G_HM(TA, TO)                                                                                                        \
  do {                                                                                                                         \
    if (nb == 1)                                                                                                               \
      heads_mfma_kernel<TA, TO, 1, 4><<<mgrid, 4 * kWave, 0, s>>>(static_cast<const TA*>(a), a_row, a_head, wp,                \
                                                                  static_cast<TO*>(out), o_row, o_head, m, n, k);              \
    else                                                                                                                       \
      heads_mfma_kernel<TA, TO, 4, 1><<<mgrid, kWave, 0, s>>>(static_cast<const TA*>(a), a_row, a_head, wp,                    \
                                                              static_cast<TO*>(out), o_row, o_head, m, n, k);                  \
  } while (0)
    if (a_dtype == kBF16 && out_dtype == kF32) BC4G_HM(bf16_t, float);
    else if (a_dtype == kBF16) BC4G_HM(bf16_t, bf16_t);
    else if (out_dtype == kF32) BC4G_HM(float, float);
    else BC4G_HM(float, bf16_t);
#undef BC4G_HM
    return check_launch("heads_gemm");
  }
  dim3 grid(ceil_div(m, kHT), ceil_div(n, kHT), heads);
#define BC4G_HG(TA, TW, TO)                                                                                              \
  heads_gemm_kernel<TA, TW, TO><<<grid, 256, 0, s>>>(static_cast<const TA*>(a), a_row, a_head, static_cast<const TW*>(w), \
                                                     static_cast<TO*>(out), o_row, o_head, m, n, k)
  const int code = a_dtype * 4 + w_dtype * 2 + out_dtype;
  BC4G_REQUIRE(a_dtype >= 0 && a_dtype <= 1 && w_dtype >= 0 && w_dtype <= 1 && out_dtype >= 0 && out_dtype <= 1,
               "heads_gemm: unknown dtypes %d, %d, %d", a_dtype, w_dtype, out_dtype);
  switch (code) {
    case 0: BC4G_HG(float, float, float); break;
    case 1: BC4G_HG(float, float, bf16_t); break;
    case 2: BC4G_HG(float, bf16_t, float); break;
    case 3: BC4G_HG(float, bf16_t, bf16_t); break;
    case 4: BC4G_HG(bf16_t, float, float); break;
    case 5: BC4G_HG(bf16_t, float, bf16_t); break;
    case 6: BC4G_HG(bf16_t, bf16_t, float); break;
    default: BC4G_HG(bf16_t, bf16_t, bf16_t); break;
  }
#undef BC4G_HG
  return check_launch("heads_gemm");
}

extern "C" int bc4g_attention_latent(const float* q_lat, float* out, const void* cache, int dtype, const float* sink,
                                     const int32_t* block_table, int table_stride, const int32_t* row_seq,
                                     const int32_t* positions, int n_rows, int heads, int rank, int rot, int page_tokens,
                                     int window, float scale, void* stream) {
  BC4G_REQUIRE(n_rows >= 0 && heads > 0 && rank > 0 && rot >= 0, "attention_latent: bad sizes T=%d heads=%d rank=%d rot=%d",
               n_rows, heads, rank, rot);
  BC4G_REQUIRE(rank + rot <= kMaxLatentRow, "attention_latent: a cache row of %d numbers is beyond %d", rank + rot, kMaxLatentRow);
  BC4G_REQUIRE(page_tokens > 0 && table_stride > 0 && window >= 0, "attention_latent: bad cache sizes page_tokens=%d "
               "table_stride=%d window=%d", page_tokens, table_stride, window);
  BC4G_REQUIRE(q_lat && out && cache && block_table && row_seq && positions, "attention_latent: a tensor is missing");
  if (n_rows == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int group = heads < kHeadsPerGroup ? heads : kHeadsPerGroup;
  BC4G_REQUIRE(ceil_div(heads, group) <= 65535, "attention_latent: %d heads are beyond the grid limit", heads);
  dim3 grid(n_rows, ceil_div(heads, group));
  const size_t lds = (static_cast<size_t>(group) * (rank + rot) + group * kWave + kWave * kTilePad) * sizeof(float);
  if (dtype == kF32)
    attention_latent_kernel<float><<<grid, group * kWave, lds, s>>>(q_lat, out, static_cast<const float*>(cache), sink, block_table,
                                                                    table_stride, row_seq, positions, heads, rank, rank + rot,
                                                                    page_tokens, window, scale);
  else if (dtype == kBF16)
    attention_latent_kernel<bf16_t><<<grid, group * kWave, lds, s>>>(q_lat, out, static_cast<const bf16_t*>(cache), sink,
                                                                     block_table, table_stride, row_seq, positions, heads, rank,
                                                                     rank + rot, page_tokens, window, scale);
  else return fail("attention_latent: unknown dtype %d", dtype);
  return check_launch("attention_latent");
}
