// Latent attention on the matrix cores (bfloat16 cache; see attention_latent.hip for what is computed).
//
// All heads read the same cache rows, so the 16 columns of a matrix-core tile are (token, head) pairs of one request:
// hb = min(heads, 16) heads of 16 / hb consecutive tokens.  A wave takes one such tile, a workgroup four tiles that
// follow each other (the head groups of one token block first, then the next token block), and the four walk the
// request's keys together: a tile of 32 cache rows goes into LDS once for all of them.
//
//   scores   S^T[keys x queries] = K[keys x row] Q^T[row x queries]: the cache rows are the A operand as they lie in
//            LDS (16 bytes a lane), the queries the B operand, kept in registers for the whole walk; a lane then
//            holds, for its query, eight of the 32 keys, so maximum and sum of a query are in-lane plus two lane swaps
//   output   O^T[latent x queries] += V^T[latent x keys] P^T[keys x queries] with V = the first `rank` numbers of the
//            same LDS rows: the weights go from the score registers straight into the B operand (which key a k-slot
//            stands for is free, as long as A agrees); the A operand wants eight keys of one latent number side by
//            side, so the latent part of a tile is kept a second time in LDS, transposed ([number][key]), written
//            two bytes at a time while the tile is staged and read eight bytes at a time (gathering the keys from the
//            rows themselves, two bytes a read, made the walk wait for LDS 256 times a tile)
//
// The keys may be cut into n_splits parts over workgroups (few rows over a long context: a decode step), whose
// unnormalised float partials a second kernel merges; the sink joins the sum where the sum is finished.
#include <float.h>
#include <math.h>

#include "api.h"
#include "common.h"
#include "mfma.h"

namespace bc4g {
namespace {

constexpr int kKeys = 32;                   // cache rows a key tile holds
constexpr int kVtPitch = 36;                // 16-bit elements of a row of the transposed latent part (32 keys and a pad)
constexpr float kLog2e = 1.4426950408889634f;

__device__ inline unsigned pack_bf16(float lo, float hi) {
  return static_cast<unsigned>(bf16_bits_from_float(lo)) | (static_cast<unsigned>(bf16_bits_from_float(hi)) << 16);
}

// KS: k-steps of 32 over a cache row (dk <= 32 KS); DB: blocks of 16 over the latent (rank <= 16 DB).
template <int KS, int DB>
__global__ __launch_bounds__(256, 2) void latent_mfma_kernel(
    const float* __restrict__ q_lat, float* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml,
    const bf16_t* __restrict__ cache, const float* __restrict__ sink, const int32_t* __restrict__ block_table,
    int table_stride, const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_ctx, int n_tokens, int heads,
    int rank, int dk, int page_tokens, int window, float scale, int hb, int tpt, int n_hg, int n_splits) {
  extern __shared__ uint4 tile[];                             // [kKeys][dk / 8 + 1] pieces of 16 bytes, then the transposed part
  const int s = blockIdx.y, z = blockIdx.z;
  const int tok0 = seq_start[s], n_tok = seq_start[s + 1] - tok0, cached = seq_ctx[s];
  const int n_tb = (n_tok + tpt - 1) / tpt, n_tiles = n_tb * n_hg;
  // (the grid's first workgroups take a request's last rows: their walks over the keys are the longest, and the short
  // ones fill in behind them)
  const int tile0 = (gridDim.x - 1 - blockIdx.x) * 4;
  if (tile0 >= n_tiles) return;                               // (the whole workgroup)
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int my_tile = tile0 + wave;
  const bool wave_live = my_tile < n_tiles;
  const int tb = wave_live ? my_tile / n_hg : 0, hg = wave_live ? my_tile % n_hg : 0;
  const int c = lane % 16, g = lane / 16;
  const int tq = tb * tpt + c / hb, head = hg * hb + c % hb;
  const bool q_live = wave_live && c / hb < tpt && tq < n_tok && head < heads;
  const int pos = cached + tq;
  const int32_t* table = block_table + static_cast<long>(s) * table_stride;
  const int cpr = dk / 8, pitch = cpr + 1;                    // 16-byte pieces of a row; of a row in LDS

  // the keys this workgroup's rows see, in tiles aligned to multiples of 32, and this part's share of them
  const int tb_last = min(n_tb - 1, (tile0 + 3) / n_hg);
  const int last_pos = cached + min(n_tok, (tb_last + 1) * tpt) - 1;
  const int first_pos = window > 0 ? max(0, cached + (tile0 / n_hg) * tpt - window + 1) : 0;
  const int kt_begin = first_pos / kKeys, kt_end = last_pos / kKeys + 1;
  const int per = (kt_end - kt_begin + n_splits - 1) / n_splits;
  const int kt_lo = kt_begin + z * per, kt_hi = min(kt_end, kt_lo + per);

  uint4 qf[KS];
  {
    const float* qrow = q_lat + (static_cast<long>(tok0 + tq) * heads + head) * dk;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      qf[ks] = zero16();
      if (q_live && ks * 32 < dk) {
        const float4 a = *reinterpret_cast<const float4*>(qrow + ks * 32 + 8 * g);
        const float4 b = *reinterpret_cast<const float4*>(qrow + ks * 32 + 8 * g + 4);
        qf[ks] = make_uint4(pack_bf16(a.x, a.y), pack_bf16(a.z, a.w), pack_bf16(b.x, b.y), pack_bf16(b.z, b.w));
      }
    }
  }
  floatx4 acc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) acc[db] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  const float scale2 = scale * kLog2e;                        // exponents to the base 2
  uint16_t* vt = reinterpret_cast<uint16_t*>(tile + kKeys * pitch);     // [rank][kVtPitch]: the latent part, transposed

  // Staging: eight threads a key, each with every eighth 16-byte piece of its row -- one look at the block table a
  // thread and tile, all of a thread's loads asked for together, and the next tile's asked for before this tile is
  // worked on, so that they are under way meanwhile (the barriers wait for LDS only).
  constexpr int kPieces = (KS * 4 + 7) / 8;
  const int st_key = threadIdx.x / 8, st_sub = threadIdx.x % 8;
  uint4 stage[kPieces];
  auto fetch = [&](int kt) {
    const int j = kt * kKeys + st_key;
    const bool there = j >= first_pos && j <= last_pos;
    const bf16_t* src = cache;
    if (there) src = cache + (static_cast<long>(table[j / page_tokens]) * page_tokens + j % page_tokens) * dk;
#pragma unroll
    for (int p = 0; p < kPieces; ++p) {
      const int part = st_sub + 8 * p;
      stage[p] = there && part < cpr ? load16(src + part * 8) : zero16();
    }
  };
  for (int kt = kt_lo; kt < kt_hi; ++kt) {
    const int j0 = kt * kKeys;
    fetch(kt);
#pragma unroll
    for (int p = 0; p < kPieces; ++p) {
      const int part = st_sub + 8 * p;
      if (part < cpr) tile[st_key * pitch + part] = stage[p];
      if (part * 8 < rank) {
        uint16_t* to = vt + part * 8 * kVtPitch + st_key;
        const unsigned w[4] = {stage[p].x, stage[p].y, stage[p].z, stage[p].w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          to[(2 * e) * kVtPitch] = static_cast<uint16_t>(w[e] & 0xffffu);
          to[(2 * e + 1) * kVtPitch] = static_cast<uint16_t>(w[e] >> 16);
        }
      }
    }
    lds_barrier();
    if (wave_live) {
    floatx4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (ks * 32 < dk) {
        s0 = mfma_16x16x32(tile[c * pitch + ks * 4 + g], qf[ks], s0);
        s1 = mfma_16x16x32(tile[(16 + c) * pitch + ks * 4 + g], qf[ks], s1);
      }
    }
    // this lane's eight keys of its query: j0 + 4g + i and j0 + 16 + 4g + i
    float p[8];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int j = j0 + (i < 4 ? 0 : 16) + 4 * g + (i & 3);
      const bool seen = q_live && j <= pos && (window == 0 || j > pos - window);
      p[i] = seen ? (i < 4 ? s0[i] : s1[i - 4]) * scale2 : -INFINITY;
      mx = fmaxf(mx, p[i]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, kWave));
    mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
    const float m_new = fmaxf(m, mx);
    const float alpha = m_new == -INFINITY ? 1.f : __builtin_amdgcn_exp2f(m - m_new);     // (m = -inf: 0)
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      p[i] = p[i] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(p[i] - m_new);
      sum += p[i];
    }
    l = l * alpha + sum;
    m = m_new;
    if (__any(alpha != 1.f)) {
#pragma unroll
      for (int db = 0; db < DB; ++db) acc[db] *= alpha;
    }
    const uint4 pf = make_uint4(pack_bf16(p[0], p[1]), pack_bf16(p[2], p[3]), pack_bf16(p[4], p[5]), pack_bf16(p[6], p[7]));
    const uint16_t* col = vt + c * kVtPitch + 4 * g;          // latent number c of a block, keys 4g .. 4g + 3
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      if (db * 16 < rank) {
        const uint2 lo = *reinterpret_cast<const uint2*>(col + db * 16 * kVtPitch);
        const uint2 hi = *reinterpret_cast<const uint2*>(col + db * 16 * kVtPitch + 16);
        const uint4 a = make_uint4(lo.x, lo.y, hi.x, hi.y);
        acc[db] = mfma_16x16x32(a, pf, acc[db]);
      }
    }
    }
    lds_barrier();                                            // the tile has been read by everyone
  }
  if (!q_live) return;
  l += __shfl_xor(l, 16, kWave);
  l += __shfl_xor(l, 32, kWave);
  const long row = static_cast<long>(tok0 + tq) * heads + head;
  if (n_splits == 1) {
    if (sink) l += __builtin_amdgcn_exp2f(sink[head] * kLog2e - m);
    const float inv = 1.0f / l;
    float* o = out + row * rank;
#pragma unroll
    for (int db = 0; db < DB; ++db)
      if (db * 16 < rank)
        *reinterpret_cast<float4*>(o + db * 16 + 4 * g) = make_float4(acc[db][0] * inv, acc[db][1] * inv, acc[db][2] * inv, acc[db][3] * inv);
  } else {
    float* o = part_o + (static_cast<long>(z) * n_tokens * heads + row) * rank;
#pragma unroll
    for (int db = 0; db < DB; ++db)
      if (db * 16 < rank)
        *reinterpret_cast<float4*>(o + db * 16 + 4 * g) = make_float4(acc[db][0], acc[db][1], acc[db][2], acc[db][3]);
    if (g == 0) {
      float* ml = part_ml + (static_cast<long>(z) * n_tokens * heads + row) * 2;
      ml[0] = m;
      ml[1] = l;
    }
  }
}

// The form in which G waves cut one tile's work between them -- wave w of a tile the k-steps w, w + G, ... of the
// scores (the partial scores are added up through LDS, every wave in the same order, so all hold the same bits and
// take the same maximum and sum) and the blocks w, w + G, ... of the latent for the output.  A wave then keeps 1 / G of
// the queries and of the sums in registers, and a tile's chain of LDS reads and matrix instructions is that much
// shorter.  A workgroup has WAVES waves and WAVES / G tiles that follow each other.  Four waves on one tile serve a
// decode step (a request's one row of up to sixteen heads is one tile).  (Eight waves on four tiles, two a tile, spill
// nothing and were tried for prompts: no faster at 16 heads and slower at 32 than the form above -- its 90 KB of LDS
// leave one workgroup a CU, whose eight waves then all wait at the same barriers, where two workgroups of the form
// above stage and compute beside each other.)
template <int KS, int DB, int G, int WAVES>
__global__ __launch_bounds__(kWave * WAVES) void latent_mfma_shared_kernel(
    const float* __restrict__ q_lat, float* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml,
    const bf16_t* __restrict__ cache, const float* __restrict__ sink, const int32_t* __restrict__ block_table,
    int table_stride, const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_ctx, int n_tokens, int heads,
    int rank, int dk, int page_tokens, int window, float scale, int hb, int tpt, int n_hg, int n_splits) {
  extern __shared__ uint4 tile[];                             // the tile, its latent part transposed, the partial scores
  constexpr int KW = (KS + G - 1) / G, DW = (DB + G - 1) / G;   // k-steps and latent blocks of a wave
  constexpr int TILES = WAVES / G, SUBS = 2 * WAVES;            // tiles of a workgroup; threads that stage one key
  const int s = blockIdx.y, z = blockIdx.z;
  const int tok0 = seq_start[s], n_tok = seq_start[s + 1] - tok0, cached = seq_ctx[s];
  const int n_tb = (n_tok + tpt - 1) / tpt, n_tiles = n_tb * n_hg;
  // (the grid's first workgroups take a request's last rows: their walks over the keys are the longest)
  const int tile0 = (gridDim.x - 1 - blockIdx.x) * TILES;
  if (tile0 >= n_tiles) return;                               // (the whole workgroup)
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int my_tile = tile0 + wave / G, part_of_tile = wave % G;
  const bool wave_live = my_tile < n_tiles;
  const int tb = wave_live ? my_tile / n_hg : 0, hg = wave_live ? my_tile % n_hg : 0;
  const int c = lane % 16, g = lane / 16;
  const int tq = tb * tpt + c / hb, head = hg * hb + c % hb;
  const bool q_live = wave_live && c / hb < tpt && tq < n_tok && head < heads;
  const int pos = cached + tq;
  const int32_t* table = block_table + static_cast<long>(s) * table_stride;
  const int cpr = dk / 8, pitch = cpr + 1;
  const int tb_last = min(n_tb - 1, (tile0 + TILES - 1) / n_hg);
  const int last_pos = cached + min(n_tok, (tb_last + 1) * tpt) - 1;
  const int first_pos = window > 0 ? max(0, cached + (tile0 / n_hg) * tpt - window + 1) : 0;
  const int kt_begin = first_pos / kKeys, kt_end = last_pos / kKeys + 1;
  const int per = (kt_end - kt_begin + n_splits - 1) / n_splits;
  const int kt_lo = kt_begin + z * per, kt_hi = min(kt_end, kt_lo + per);

  uint4 qf[KW];
  {
    const float* qrow = q_lat + (static_cast<long>(tok0 + tq) * heads + head) * dk;
#pragma unroll
    for (int i = 0; i < KW; ++i) {
      const int ks = part_of_tile + G * i;
      qf[i] = zero16();
      if (q_live && ks * 32 < dk) {
        const float4 a = *reinterpret_cast<const float4*>(qrow + ks * 32 + 8 * g);
        const float4 b = *reinterpret_cast<const float4*>(qrow + ks * 32 + 8 * g + 4);
        qf[i] = make_uint4(pack_bf16(a.x, a.y), pack_bf16(a.z, a.w), pack_bf16(b.x, b.y), pack_bf16(b.z, b.w));
      }
    }
  }
  floatx4 acc[DW];
#pragma unroll
  for (int i = 0; i < DW; ++i) acc[i] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  const float scale2 = scale * kLog2e;
  uint16_t* vt = reinterpret_cast<uint16_t*>(tile + kKeys * pitch);
  float4* partial = reinterpret_cast<float4*>(reinterpret_cast<char*>(tile) + kKeys * pitch * 16 + ((rank * kVtPitch * 2 + 15) / 16) * 16);

  // Staging: SUBS threads a key, each with every SUBS-th 16-byte piece of its row -- one look at the block table a
  // thread and tile, all of a thread's loads asked for together.
  constexpr int kPieces = (KS * 4 + SUBS - 1) / SUBS;
  const int st_key = threadIdx.x / SUBS, st_sub = threadIdx.x % SUBS;
  uint4 stage[kPieces];
  for (int kt = kt_lo; kt < kt_hi; ++kt) {
    const int j0 = kt * kKeys;
    {
      const int j = j0 + st_key;
      const bool there = j >= first_pos && j <= last_pos;
      const bf16_t* src = cache;
      if (there) src = cache + (static_cast<long>(table[j / page_tokens]) * page_tokens + j % page_tokens) * dk;
#pragma unroll
      for (int p = 0; p < kPieces; ++p) {
        const int part = st_sub + SUBS * p;
        stage[p] = there && part < cpr ? load16(src + part * 8) : zero16();
      }
    }
#pragma unroll
    for (int p = 0; p < kPieces; ++p) {
      const int part = st_sub + SUBS * p;
      if (part < cpr) tile[st_key * pitch + part] = stage[p];
      if (part * 8 < rank) {
        uint16_t* to = vt + part * 8 * kVtPitch + st_key;
        const unsigned w[4] = {stage[p].x, stage[p].y, stage[p].z, stage[p].w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          to[(2 * e) * kVtPitch] = static_cast<uint16_t>(w[e] & 0xffffu);
          to[(2 * e + 1) * kVtPitch] = static_cast<uint16_t>(w[e] >> 16);
        }
      }
    }
    lds_barrier();
    floatx4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
    if (wave_live) {
#pragma unroll
      for (int i = 0; i < KW; ++i) {
        const int ks = part_of_tile + G * i;
        if (ks * 32 < dk) {
          s0 = mfma_16x16x32(tile[c * pitch + ks * 4 + g], qf[i], s0);
          s1 = mfma_16x16x32(tile[(16 + c) * pitch + ks * 4 + g], qf[i], s1);
        }
      }
    }
    partial[(wave * kWave + lane) * 2] = make_float4(s0[0], s0[1], s0[2], s0[3]);
    partial[(wave * kWave + lane) * 2 + 1] = make_float4(s1[0], s1[1], s1[2], s1[3]);
    lds_barrier();
    if (wave_live) {
      float p[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) p[i] = 0.f;
#pragma unroll
      for (int w = 0; w < G; ++w) {                           // (in this order in every wave of the tile)
        const int from = ((wave / G) * G + w) * kWave + lane;
        const float4 a = partial[from * 2], b = partial[from * 2 + 1];
        p[0] += a.x, p[1] += a.y, p[2] += a.z, p[3] += a.w, p[4] += b.x, p[5] += b.y, p[6] += b.z, p[7] += b.w;
      }
      float mx = -INFINITY;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int j = j0 + (i < 4 ? 0 : 16) + 4 * g + (i & 3);
        const bool seen = q_live && j <= pos && (window == 0 || j > pos - window);
        p[i] = seen ? p[i] * scale2 : -INFINITY;
        mx = fmaxf(mx, p[i]);
      }
      mx = fmaxf(mx, __shfl_xor(mx, 16, kWave));
      mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
      const float m_new = fmaxf(m, mx);
      const float alpha = m_new == -INFINITY ? 1.f : __builtin_amdgcn_exp2f(m - m_new);
      float sum = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        p[i] = p[i] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(p[i] - m_new);
        sum += p[i];
      }
      l = l * alpha + sum;
      m = m_new;
      if (__any(alpha != 1.f)) {
#pragma unroll
        for (int i = 0; i < DW; ++i) acc[i] *= alpha;
      }
      const uint4 pf = make_uint4(pack_bf16(p[0], p[1]), pack_bf16(p[2], p[3]), pack_bf16(p[4], p[5]), pack_bf16(p[6], p[7]));
      const uint16_t* col = vt + c * kVtPitch + 4 * g;
#pragma unroll
      for (int i = 0; i < DW; ++i) {
        const int db = part_of_tile + G * i;
        if (db * 16 < rank) {
          const uint2 lo = *reinterpret_cast<const uint2*>(col + db * 16 * kVtPitch);
          const uint2 hi = *reinterpret_cast<const uint2*>(col + db * 16 * kVtPitch + 16);
          acc[i] = mfma_16x16x32(make_uint4(lo.x, lo.y, hi.x, hi.y), pf, acc[i]);
        }
      }
    }
    lds_barrier();                                            // the tile has been read by everyone
  }
  if (!q_live) return;
  l += __shfl_xor(l, 16, kWave);
  l += __shfl_xor(l, 32, kWave);
  const long row = static_cast<long>(tok0 + tq) * heads + head;
  float inv = 1.f;
  float* o = part_o + (static_cast<long>(z) * n_tokens * heads + row) * rank;
  if (n_splits == 1) {
    if (sink) l += __builtin_amdgcn_exp2f(sink[head] * kLog2e - m);
    inv = 1.0f / l;
    o = out + row * rank;
  } else if (part_of_tile == 0 && g == 0) {
    float* ml = part_ml + (static_cast<long>(z) * n_tokens * heads + row) * 2;
    ml[0] = m;
    ml[1] = l;
  }
#pragma unroll
  for (int i = 0; i < DW; ++i) {
    const int db = part_of_tile + G * i;
    if (db * 16 < rank)
      *reinterpret_cast<float4*>(o + db * 16 + 4 * g) = make_float4(acc[i][0] * inv, acc[i][1] * inv, acc[i][2] * inv, acc[i][3] * inv);
  }
}

// out[row] = sum_z part_o[z][row] 2^(m_z - M) / (sum_z l_z 2^(m_z - M) + 2^(sink log2(e) - M)): a workgroup a (row, head).
// Its first wave weighs the parts (a lane a part: at most 64), then a thread takes four numbers of the latent and asks
// for eight parts of them at a time.
constexpr int kMergeBlock = 128;
__global__ __launch_bounds__(kMergeBlock) void latent_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                                   const float* __restrict__ sink, float* __restrict__ out,
                                                                   long rows, int heads, int rank, int n_splits) {
  __shared__ float weight[kWave + 1];
  const long row = blockIdx.x;
  if (threadIdx.x < kWave) {
    const int lane = threadIdx.x;
    float mz = -INFINITY, lz = 0.f;
    if (lane < n_splits) {
      const float2 ml = *reinterpret_cast<const float2*>(part_ml + (lane * rows + row) * 2);
      mz = ml.x, lz = ml.y;
    }
    const float big = wave_max(mz);
    const float wz = __builtin_amdgcn_exp2f(mz - big);
    const float total = wave_sum(lz * wz) + (sink ? __builtin_amdgcn_exp2f(sink[row % heads] * kLog2e - big) : 0.f);
    weight[lane] = wz;
    if (lane == 0) weight[kWave] = 1.0f / total;
  }
  __syncthreads();
  const float inv = weight[kWave];
  for (int d = 4 * threadIdx.x; d < rank; d += 4 * kMergeBlock) {
    float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll 8
    for (int z = 0; z < n_splits; ++z) {
      const float4 v = *reinterpret_cast<const float4*>(part_o + (z * rows + row) * rank + d);
      const float wz = weight[z];
      sum.x = fmaf(v.x, wz, sum.x), sum.y = fmaf(v.y, wz, sum.y), sum.z = fmaf(v.z, wz, sum.z), sum.w = fmaf(v.w, wz, sum.w);
    }
    *reinterpret_cast<float4*>(out + row * rank + d) = make_float4(sum.x * inv, sum.y * inv, sum.z * inv, sum.w * inv);
  }
}

}  // namespace
}  // namespace bc4g

using namespace bc4g;

// Whether the matrix-core kernel takes these sizes (a bfloat16 cache): cache rows of whole k-steps, a latent of whole
// blocks, both within what a wave's registers hold.
extern "C" int bc4g_attention_latent_mfma_takes(int rank, int rot) {
  const int dk = rank + rot;
  return dk % 32 == 0 && rank % 16 == 0 && dk <= 576 && rank <= 512 && rank > 0;
}

// q_lat [T, heads, rank + rot] float32; out [T, heads, rank] float32; cache bfloat16 [pages, page_tokens, rank + rot].
// n_tiles_most: the most (token block, head group) tiles a request of the step has; n_splits > 1 needs part_o
// [n_splits, T, heads, rank] and part_ml [n_splits, T, heads, 2].
extern "C" int bc4g_attention_latent_mfma(const float* q_lat, float* out, float* part_o, float* part_ml, const void* cache,
                                          const float* sink, const int32_t* block_table, int table_stride,
                                          const int32_t* seq_start, const int32_t* seq_ctx, int n_seqs, int n_tokens,
                                          int most_tokens, int heads, int rank, int rot, int page_tokens, int window,
                                          float scale, int n_splits, void* stream) {
  BC4G_REQUIRE(n_seqs >= 0 && n_tokens >= 0 && heads > 0 && most_tokens >= 0 && bc4g_attention_latent_mfma_takes(rank, rot),
               "attention_latent_mfma: sizes it does not take (S=%d T=%d heads=%d rank=%d rot=%d)", n_seqs, n_tokens, heads, rank, rot);
  BC4G_REQUIRE(page_tokens > 0 && table_stride > 0 && window >= 0 && n_splits >= 1 && n_splits <= 64,
               "attention_latent_mfma: bad cache sizes or parts (page_tokens=%d table_stride=%d window=%d parts=%d)", page_tokens,
               table_stride, window, n_splits);
  BC4G_REQUIRE(q_lat && out && cache && block_table && seq_start && seq_ctx && (n_splits == 1 || (part_o && part_ml)),
               "attention_latent_mfma: a tensor is missing");
  BC4G_REQUIRE(reinterpret_cast<uintptr_t>(cache) % 16 == 0 && reinterpret_cast<uintptr_t>(q_lat) % 16 == 0 &&
               reinterpret_cast<uintptr_t>(out) % 16 == 0, "attention_latent_mfma: operands must lie on 16-byte boundaries");
  if (n_tokens == 0 || n_seqs == 0 || most_tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int dk = rank + rot;
  const int hb = heads < 16 ? heads : 16, tpt = 16 / hb, n_hg = ceil_div(heads, hb);
  const int most_tiles = ceil_div(most_tokens, tpt) * n_hg;
  BC4G_REQUIRE(n_seqs <= 65535 && n_splits <= 65535, "attention_latent_mfma: %d requests are beyond the grid limit", n_seqs);
  // no request with four tiles (a decode step): a workgroup a tile, four waves on it; else four tiles a workgroup, a
  // wave on each
  const bool one_tile = most_tiles < 4;
  dim3 grid(one_tile ? most_tiles : ceil_div(most_tiles, 4), n_seqs, n_splits);
  const size_t lds = static_cast<size_t>(kKeys) * (dk / 8 + 1) * 16 + (static_cast<size_t>(rank) * kVtPitch * 2 + 15) / 16 * 16 +
                     (one_tile ? 4 * kWave * 32 : 0);
  const bf16_t* kc = static_cast<const bf16_t*>(cache);
  // (more than 64 KB of LDS a workgroup has to be asked for, once for a kernel: the most this kernel ever takes)
#define BC4G_LATENT(KS, DB)                                                                                                 \
  static const hipError_t allowed = hipFuncSetAttribute(reinterpret_cast<const void*>(&latent_mfma_kernel<KS, DB>),         \
                                                        hipFuncAttributeMaxDynamicSharedMemorySize,                          \
                                                        kKeys * (KS * 4 + 1) * 16 + DB * 16 * kVtPitch * 2);                 \
  static const hipError_t allowed4 = hipFuncSetAttribute(                                                                    \
      reinterpret_cast<const void*>(&latent_mfma_shared_kernel<KS, DB, 4, 4>), hipFuncAttributeMaxDynamicSharedMemorySize,   \
      kKeys * (KS * 4 + 1) * 16 + DB * 16 * kVtPitch * 2 + 4 * kWave * 32);                                                  \
  BC4G_REQUIRE(allowed == hipSuccess && allowed4 == hipSuccess,                                                              \
               "attention_latent_mfma: %zu bytes of LDS a workgroup are refused", lds);                                       \
  if (one_tile)                                                                                                               \
    latent_mfma_shared_kernel<KS, DB, 4, 4><<<grid, 4 * kWave, lds, s>>>(q_lat, out, part_o, part_ml, kc, sink, block_table,  \
                                                                         table_stride, seq_start, seq_ctx, n_tokens, heads, rank, \
                                                                         dk, page_tokens, window, scale, hb, tpt, n_hg, n_splits); \
  else                                                                                                                        \
    latent_mfma_kernel<KS, DB><<<grid, 256, lds, s>>>(q_lat, out, part_o, part_ml, kc, sink, block_table, table_stride, seq_start, \
                                                      seq_ctx, n_tokens, heads, rank, dk, page_tokens, window, scale, hb, tpt, n_hg, \
                                                      n_splits)
  if (dk <= 128 && rank <= 64) { BC4G_LATENT(4, 4); }
  else if (dk <= 320 && rank <= 256) { BC4G_LATENT(10, 16); }
  else { BC4G_LATENT(18, 32); }
#undef BC4G_LATENT
  if (n_splits > 1)
    latent_merge_kernel<<<static_cast<unsigned>(static_cast<long>(n_tokens) * heads), kMergeBlock, 0, s>>>(
        part_o, part_ml, sink, out, static_cast<long>(n_tokens) * heads, heads, rank, n_splits);
  return check_launch("attention_latent_mfma");
}
