// Attention through low-rank latents.  Per token one vector is cached for all heads: the
// normalised latent c [rank] followed by one rotated key part [dr].  A head's key is
// [W_uk,h c | rotated part] and its value W_uv,h c, so with the query's unrotated part folded
// through W_uk,h (q' = W_uk,h^T q, [rank]) the score is q' . c + q_rot . k_rot, the weighted
// sum over the keys is taken of c itself, and W_uv,h is applied once to that sum:
//
//   latent_kv_append   sums of W_dkv h -> RMS norm (weights) of the first rank, rotation of the
//                      last dr (halves paired), appended to the pages (one row of rank + dr a slot)
//   latent_query       sums of W_uq c_q -> per head [W_uk,h^T q_h | rotated q_h], rank + dr wide
//   attn_latent        one workgroup a (token, head): online softmax over 256 keys at a time,
//                      the values being the first rank elements of the cached rows
//   latent_out         per head W_uv,h times the attended latent, times sigmoid of the gate's sums
//
// Scores, softmax, norms and rotation are 32-bit; the cached rows, the folded queries and the
// attended latents are stored in the compute type.
//
// A page holds its slots' rows [slot][rank + dr] and then the latents once more, transposed
// [rank][slot]: the weighted sum over the keys runs along the slots, and the matrix cores want
// the dimension that is summed over contiguous.  attn_latent has two kernels: one workgroup a
// (token, head) in 32-bit arithmetic for every size and type, and, in bfloat16 for ranks in
// steps of 16 and rows in steps of 8, one on the matrix cores (below).
#include <math.h>
#include <stdint.h>

#include "common.hpp"
#include "kllm_kernels.h"

namespace kllm {

constexpr int kLatThreads = 256;
constexpr int kLatMaxRow = 1024;       // rank + dr of a cached row
constexpr int kLatMaxPer = kLatMaxRow / kLatThreads;

template <typename T>
__global__ __launch_bounds__(kLatThreads) void latent_kv_append_kernel(
    const float* __restrict__ dkv, int nsplit, long split_stride, const float* __restrict__ weight, float eps,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, T* __restrict__ cache,
    const int* __restrict__ positions, const int* __restrict__ span_of_token, const int* __restrict__ block_table,
    int max_pages, int page_size, int rank, int dr, long in_stride) {
  __shared__ float red[16];
  const long t = blockIdx.x;
  const int tid = threadIdx.x;
  const int row = rank + dr, half = dr / 2;
  const float* in = dkv + t * in_stride;
  const int pos = positions[t];
  const long page = block_table[(long)span_of_token[t] * max_pages + pos / page_size];
  const long page_elems = (long)page_size * (row + rank);
  const int slot = pos % page_size;
  T* dst = cache + page * page_elems + (long)slot * row;
  T* dst_t = cache + page * page_elems + (long)page_size * row + slot;     // [rank][slot]
  float v[kLatMaxPer];
  float ss = 0.f;
#pragma unroll
  for (int q = 0; q < kLatMaxPer; ++q) {
    const int i = tid + q * kLatThreads;
    v[q] = 0.f;
    if (i < rank) {
      for (int s = 0; s < nsplit; ++s) v[q] += in[s * split_stride + i];
      ss = fmaf(v[q], v[q], ss);
    }
  }
  const float rstd = 1.f / sqrtf(block_sum(ss, red) / (float)rank + eps);
#pragma unroll
  for (int q = 0; q < kLatMaxPer; ++q) {
    const int i = tid + q * kLatThreads;
    if (i < rank) {
      const T c = from_f32<T>(v[q] * rstd * weight[i]);
      dst[i] = c;
      dst_t[(long)i * page_size] = c;
    }
  }
  for (int i = tid; i < half; i += kLatThreads) {
    float a = 0.f, b = 0.f;
    for (int s = 0; s < nsplit; ++s) {
      a += in[s * split_stride + rank + i];
      b += in[s * split_stride + rank + half + i];
    }
    const float c = cos_t[t * half + i], sn = sin_t[t * half + i];
    dst[rank + i] = from_f32<T>(a * c - b * sn);
    dst[rank + half + i] = from_f32<T>(b * c + a * sn);
  }
}

// out [n][r] = N(in row's r elements) * weight, the rows of `in` in_stride apart; one workgroup a row.
template <typename T>
__global__ __launch_bounds__(kLatThreads) void latent_norm_kernel(const float* __restrict__ in, int nsplit,
                                                                  long split_stride, long in_stride,
                                                                  const float* __restrict__ weight, float eps,
                                                                  T* __restrict__ out, int r) {
  __shared__ float red[16];
  const long t = blockIdx.x;
  const int tid = threadIdx.x;
  const float* src = in + t * in_stride;
  float ss = 0.f;
  for (int i = tid; i < r; i += kLatThreads) {
    float v = 0.f;
    for (int s = 0; s < nsplit; ++s) v += src[s * split_stride + i];
    ss = fmaf(v, v, ss);
  }
  const float rstd = 1.f / sqrtf(block_sum(ss, red) / (float)r + eps);
  for (int i = tid; i < r; i += kLatThreads) {
    float v = 0.f;
    for (int s = 0; s < nsplit; ++s) v += src[s * split_stride + i];
    out[t * r + i] = from_f32<T>(v * rstd * weight[i]);
  }
}

// q: [nsplit][n][H * (d + dr)], a head laid out [d unrotated | dr rotated]; w_uk [H * d][rank].
template <typename T>
__global__ __launch_bounds__(kLatThreads) void latent_query_kernel(
    const float* __restrict__ q, int nsplit, long split_stride, const T* __restrict__ w_uk,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, T* __restrict__ out, int H, int d, int dr,
    int rank) {
  extern __shared__ float qh[];          // [d + dr]
  const long t = blockIdx.x;
  const int h = blockIdx.y, tid = threadIdx.x;
  const int hw = d + dr, half = dr / 2;
  const float* in = q + (t * H + h) * hw;
  for (int i = tid; i < hw; i += kLatThreads) {
    float v = 0.f;
    for (int s = 0; s < nsplit; ++s) v += in[s * split_stride + i];
    qh[i] = v;
  }
  __syncthreads();
  T* dst = out + (t * H + h) * (rank + dr);
  const T* w = w_uk + (long)h * d * rank;
  for (int r = tid; r < rank; r += kLatThreads) {
    float acc = 0.f;
    for (int i = 0; i < d; ++i) acc = fmaf(qh[i], to_f32(w[(long)i * rank + r]), acc);
    dst[r] = from_f32<T>(acc);
  }
  for (int i = tid; i < half; i += kLatThreads) {
    const float a = qh[d + i], b = qh[d + half + i];
    const float c = cos_t[t * half + i], sn = sin_t[t * half + i];
    dst[rank + i] = from_f32<T>(a * c - b * sn);
    dst[rank + half + i] = from_f32<T>(b * c + a * sn);
  }
}

template <typename T>
__global__ __launch_bounds__(kLatThreads) void attn_latent_kernel(
    const T* __restrict__ q, T* __restrict__ out, const T* __restrict__ cache, const int* __restrict__ positions,
    const int* __restrict__ span_of_token, const int* __restrict__ block_table, int max_pages, int page_size, int H,
    int row, int rank, float scale) {
  __shared__ float qs[kLatMaxRow];
  __shared__ float ps[kLatThreads];
  __shared__ float red[16];
  const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const long page_elems = (long)page_size * (row + rank);
  const int len = positions[t] + 1;
  const int* table = block_table + (long)span_of_token[t] * max_pages;
  const T* qrow = q + ((long)t * H + h) * row;
  for (int i = tid; i < row; i += kLatThreads) qs[i] = to_f32(qrow[i]);
  __syncthreads();
  float m = -INFINITY, l = 0.f;
  float acc[kLatMaxPer];
#pragma unroll
  for (int c = 0; c < kLatMaxPer; ++c) acc[c] = 0.f;
  for (int base = 0; base < len; base += kLatThreads) {
    const int key = base + tid;
    float s = -INFINITY;
    if (key < len) {
      const T* krow = cache + (long)table[key / page_size] * page_elems + (long)(key % page_size) * row;
      float dot = 0.f;
      for (int i = 0; i < row; ++i) dot = fmaf(qs[i], to_f32(krow[i]), dot);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, block_max(s, red));
    const float alpha = expf(m - m_new);
    const float p = (s == -INFINITY) ? 0.f : expf(s - m_new);
    ps[tid] = p;
    l = l * alpha + block_sum(p, red);       // its barriers also publish ps
    m = m_new;
    const int nk = min(kLatThreads, len - base);
#pragma unroll
    for (int c = 0; c < kLatMaxPer; ++c) {
      const int e = tid + c * kLatThreads;
      acc[c] *= alpha;
      if (e < rank) {
        float a = acc[c];
        int pg = -1;
        const T* prow = nullptr;
        for (int k = 0; k < nk; ++k) {
          const int kk = base + k;
          if (kk / page_size != pg) {
            pg = kk / page_size;
            prow = cache + (long)table[pg] * page_elems;
          }
          a = fmaf(ps[k], to_f32(prow[(long)(kk % page_size) * row + e]), a);
        }
        acc[c] = a;
      }
    }
    __syncthreads();                         // ps is rewritten by the next round
  }
#pragma unroll
  for (int c = 0; c < kLatMaxPer; ++c) {
    const int e = tid + c * kLatThreads;
    if (e < rank) out[((long)t * H + h) * rank + e] = from_f32<T>(acc[c] / l);
  }
}

// attn_latent on the matrix cores (bfloat16).  A workgroup takes one token and up to 16 heads;
// its four waves take the token's keys in tiles of 32, round robin, and meet in LDS.  All heads
// read the same keys, so the 16 heads are the columns of one product:
// MFMA 16x16x32 (lane l: g = l/16, c = l%16): A[c][8g..8g+7], B[8g..8g+7][c], D[4g+i][c].
// Scores: A = 16 keys x 32 elements of their rows (one row per lane, straight from the page),
// B = the folded queries of the 16 heads, D[key 4g+i][head c].  Weighted sum: the 32 slots that
// are summed over are the keys (4g+j) of the tile's first half for j < 4 and of its second half for
// j >= 4, which is how a lane holds its probabilities; A = latents [element c][those keys], two
// 8-byte reads from the transposed copy.  NR: 16-element pieces of the latent a lane accumulates.
constexpr int kLatWaves = 4;

// KS: steps of 32 over a row whose pieces of the query a lane keeps in registers (0: it asks for
// them at every tile, for rows longer than the built sizes).
template <int NR, int KS>
__global__ __launch_bounds__(64 * kLatWaves) void attn_latent_mfma_kernel(
    const bf16_t* __restrict__ q, bf16_t* __restrict__ out, const bf16_t* __restrict__ cache,
    const int* __restrict__ positions, const int* __restrict__ span_of_token, const int* __restrict__ block_table,
    int max_pages, int page_size, unsigned page_magic, int H, int row, int rank, float scale, float* __restrict__ part) {
  extern __shared__ float lat_red[];            // [kLatWaves - 1][NR * 4 + 2][64]
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int g = lane / 16, c = lane % 16;
  const int t = blockIdx.x, h0 = blockIdx.y * 16;
  const int head = min(h0 + c, H - 1);
  const bool head_ok = h0 + c < H;
  const int len = positions[t] + 1;
  const int* table = block_table + (long)span_of_token[t] * max_pages;
  const long page_elems = (long)page_size * (row + rank);
  const int ksteps = (row + 31) / 32, nr = rank / 16;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  const bf16_t* qrow = q + ((long)t * H + head) * row;
  bf16x8 qreg[KS > 0 ? KS : 1];
#pragma unroll
  for (int kk = 0; kk < KS; ++kk) {
    const int d0 = 32 * kk + 8 * g;
    qreg[kk] = (d0 < row && head_ok) ? *reinterpret_cast<const bf16x8*>(qrow + d0) : zero8;
  }

  float m = -INFINITY, l = 0.f;
  floatx4 acc[NR];
#pragma unroll
  for (int r = 0; r < NR; ++r) acc[r] = floatx4{0.f, 0.f, 0.f, 0.f};

  // The tiles go in turn to the slices (workgroups of the same token and heads, blockIdx.z: where
  // tokens and heads alone leave CUs idle) and, within a slice, to the waves.
  const int nslices = gridDim.z, slice = blockIdx.z;
  const int tiles = (len + 31) / 32;
  for (int tile = slice * kLatWaves + wave; tile < tiles; tile += kLatWaves * nslices) {
    const int kb = tile * 32;
    // a half (16 keys) lies in one page (pages hold a multiple of 16 slots)
    const bf16_t* pbase[2];
    int slot0[2];
    bool live[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int k0 = kb + 16 * u;
      live[u] = k0 < len;
      const int pi = live[u] ? (int)(__umulhi((unsigned)k0, page_magic) >> 3) : 0;   // k0 / page_size (see the launch)
      const int page = table[pi];
      pbase[u] = cache + (long)page * page_elems;
      slot0[u] = live[u] ? k0 - pi * page_size : 0;
    }
    floatx4 s[2] = {floatx4{0.f, 0.f, 0.f, 0.f}, floatx4{0.f, 0.f, 0.f, 0.f}};
    auto score_step = [&](int ks, const bf16x8& qb) {
      const int d0 = 32 * ks + 8 * g;
      const bool in = d0 < row;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const bf16x8 a = (in && live[u]) ? *reinterpret_cast<const bf16x8*>(pbase[u] + (long)(slot0[u] + c) * row + d0) : zero8;
        s[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qb, s[u], 0, 0, 0);
      }
    };
    if constexpr (KS > 0) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        if (ks < ksteps) score_step(ks, qreg[ks]);
    } else {
      for (int ks = 0; ks < ksteps; ++ks) {
        const int d0 = 32 * ks + 8 * g;
        score_step(ks, (d0 < row && head_ok) ? *reinterpret_cast<const bf16x8*>(qrow + d0) : zero8);
      }
    }
    // ---- online softmax for this lane's head over its 8 keys, then over the 4 lanes of the column
    float tmax = -INFINITY;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = kb + 16 * u + 4 * g + i;
        s[u][i] = key < len ? s[u][i] * scale : -INFINITY;
        tmax = fmaxf(tmax, s[u][i]);
      }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, kWave));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, kWave));
    const float m_new = fmaxf(m, tmax);                    // finite: every tile holds a key that is read
    const float alpha = expf(m - m_new);
    bf16x8 pb;
    float psum = 0.f;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = (s[u][i] == -INFINITY) ? 0.f : expf(s[u][i] - m_new);
        const bf16_t pr = (bf16_t)p;
        pb[4 * u + i] = pr;
        psum += (float)pr;
      }
    l = l * alpha + psum;
    m = m_new;
    // ---- the weighted sum of the latents: slots beyond the last key may hold anything
    const bf16_t* vt[2] = {pbase[0] + (long)page_size * row + slot0[0] + 4 * g,
                           pbase[1] + (long)page_size * row + slot0[1] + 4 * g};
#pragma unroll
    for (int r = 0; r < NR; ++r) {
      if (r < nr) {
        acc[r] *= alpha;
        bf16x8 a;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const bf16x4 v = live[u] ? *reinterpret_cast<const bf16x4*>(vt[u] + (long)(16 * r + c) * page_size) : bf16x4{0, 0, 0, 0};
#pragma unroll
          for (int i = 0; i < 4; ++i) a[4 * u + i] = (kb + 16 * u + 4 * g + i < len) ? v[i] : (bf16_t)0.f;
        }
        acc[r] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb, acc[r], 0, 0, 0);
      }
    }
  }
  l += __shfl_xor(l, 16, kWave);
  l += __shfl_xor(l, 32, kWave);

  // ---- the waves meet: waves 1.. leave maximum, sum and output in LDS (lane-contiguous), wave 0
  // adds them in a fixed order with weights exp(m_w - max m) and writes.
  constexpr int kRows = NR * 4 + 2;
  if (wave > 0) {
    float* mine = lat_red + (long)(wave - 1) * kRows * kWave + lane;
#pragma unroll
    for (int r = 0; r < NR; ++r)
#pragma unroll
      for (int i = 0; i < 4; ++i) mine[(4 * r + i) * kWave] = acc[r][i];
    mine[(NR * 4) * kWave] = m;
    mine[(NR * 4 + 1) * kWave] = l;
  }
  __syncthreads();
  if (wave > 0 || !head_ok) return;
  float mw[kLatWaves - 1], ww[kLatWaves - 1], M = m;
#pragma unroll
  for (int w = 0; w < kLatWaves - 1; ++w) {
    mw[w] = lat_red[((long)w * kRows + NR * 4) * kWave + lane];
    M = fmaxf(M, mw[w]);
  }
  const float w0 = (m == -INFINITY) ? 0.f : expf(m - M);    // (a slice beyond the token's keys has none)
  l *= w0;
#pragma unroll
  for (int w = 0; w < kLatWaves - 1; ++w) {
    ww[w] = (mw[w] == -INFINITY) ? 0.f : expf(mw[w] - M);
    l += ww[w] * lat_red[((long)w * kRows + NR * 4 + 1) * kWave + lane];
  }
  if (nslices > 1) {
    // the slice's sums as they are, with its maximum and its sum of probabilities: rows of
    // rank + 2 floats; a slice without a key leaves a maximum of -inf and zeros
    float* prow = part + (((long)t * H + head) * nslices + slice) * (rank + 2);
#pragma unroll
    for (int r = 0; r < NR; ++r) {
      if (r < nr) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float o = acc[r][i] * w0;
#pragma unroll
          for (int w = 0; w < kLatWaves - 1; ++w) o += ww[w] * lat_red[((long)w * kRows + 4 * r + i) * kWave + lane];
          prow[16 * r + 4 * g + i] = o;
        }
      }
    }
    if (g == 0) {
      prow[rank] = M;
      prow[rank + 1] = l;
    }
    return;
  }
  const float inv = 1.f / l;
  bf16_t* orow = out + ((long)t * H + head) * rank;
#pragma unroll
  for (int r = 0; r < NR; ++r) {
    if (r < nr) {
      bf16x4 v;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float o = acc[r][i] * w0;
#pragma unroll
        for (int w = 0; w < kLatWaves - 1; ++w) o += ww[w] * lat_red[((long)w * kRows + 4 * r + i) * kWave + lane];
        v[i] = (bf16_t)(o * inv);
      }
      *reinterpret_cast<bf16x4*>(orow + 16 * r + 4 * g) = v;
    }
  }
}

// The same for steps of many tokens: a workgroup takes four consecutive tokens of the step and up
// to 16 heads, one token a wave.  Tokens of one request read the same keys: a tile of 32 keys
// (their rows, and their latents with the keys side by side) goes through LDS once for the
// four, which cuts the traffic between L2 and the CUs to a quarter.  Where the four tokens
// belong to several requests, the requests take their turns.  No merge: a wave has all keys
// of its token.  LDS: rows [32][row + 8], latents [rank][32 + 4] (padded against bank conflicts).
template <int NR, int KS>
__global__ __launch_bounds__(64 * kLatWaves) void attn_latent_block_kernel(
    const bf16_t* __restrict__ q, bf16_t* __restrict__ out, const bf16_t* __restrict__ cache,
    const int* __restrict__ positions, const int* __restrict__ span_of_token, const int* __restrict__ block_table,
    int max_pages, int page_size, unsigned page_magic, int n, int H, int row, int rank, float scale) {
  extern __shared__ __attribute__((aligned(16))) bf16_t lat_tiles[];
  // page of a key without a division: page_magic = ceil(2^35 / page_size) from the host, exact for
  // keys below 2^24 and pages of up to 2,048 slots (checked at the launch)
  auto page_index = [&](int key) { return (int)(__umulhi((unsigned)key, page_magic) >> 3); };
  const int KLD = row + 8, VLD = 36;
  bf16_t* ks = lat_tiles;                      // [32][KLD]
  bf16_t* vs = lat_tiles + 32 * KLD;           // [rank][VLD]
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int g = lane / 16, c = lane % 16;
  // later tokens of a prompt read more keys: the workgroups with the most to do start first
  const int t_first = (gridDim.x - 1 - blockIdx.x) * kLatWaves, h0 = blockIdx.y * 16;
  const int t = min(t_first + wave, n - 1);
  const bool token_ok = t_first + wave < n;
  const int head = min(h0 + c, H - 1);
  const bool head_ok = h0 + c < H;
  const int my_span = span_of_token[t];
  const int len = positions[t] + 1;
  const long page_elems = (long)page_size * (row + rank);
  const int ksteps = (row + 31) / 32, nr = rank / 16;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  const bf16_t* qrow = q + ((long)t * H + head) * row;
  const int rows_here = min(kLatWaves, n - t_first);
  bf16x8 qreg[KS > 0 ? KS : 1];
#pragma unroll
  for (int kk = 0; kk < KS; ++kk) {
    const int d0 = 32 * kk + 8 * g;
    qreg[kk] = (d0 < row && head_ok) ? *reinterpret_cast<const bf16x8*>(qrow + d0) : zero8;
  }

  float m = -INFINITY, l = 0.f;
  floatx4 acc[NR];
#pragma unroll
  for (int r = 0; r < NR; ++r) acc[r] = floatx4{0.f, 0.f, 0.f, 0.f};

  for (int first = 0; first < rows_here;) {
    const int span = span_of_token[t_first + first];
    int last = first;
    while (last + 1 < rows_here && span_of_token[t_first + last + 1] == span) ++last;
    const int group_len = positions[t_first + last] + 1;      // the group's last token reads the most keys
    const bool mine = token_ok && wave >= first && wave <= last;
    const int* table = block_table + (long)span * max_pages;
    // ---- a tile's way into LDS: 16-byte pieces (a half, 16 keys, lies in one page).  For the built
    // row sizes a thread's pieces of the NEXT tile are asked for before the products of this one
    // and wait in registers meanwhile.
    const int row8 = row / 8;
    constexpr int KP = KS / 2, VP = NR / 4;     // pieces a thread: 32 rows x 4 KS / 256, 16 NR elements x 4 / 256
    struct Stage {
      bf16x8 k[KP > 0 ? KP : 1], v[VP];
    };
    auto k_piece = [&](int i, int kb) -> bf16x8 {
      const int kr = i / row8;                                // (for the built sizes: unrolled, i and row8 known per thread before the loop)
      const int key = kb + kr;
      if (i >= 32 * row8 || key >= group_len) return zero8;
      const int pi = page_index(key);
      const long pg = table[pi];
      return *reinterpret_cast<const bf16x8*>(cache + pg * page_elems + (long)(key - pi * page_size) * row + 8 * (i - kr * row8));
    };
    auto v_piece = [&](int i, int kb) -> bf16x8 {             // 8 keys of one element
      const int e = i / 4, key = kb + 8 * (i % 4);
      if (e >= rank || key >= group_len) return zero8;
      const int pi = page_index(key);
      const long pg = table[pi];
      bf16x8 v = *reinterpret_cast<const bf16x8*>(cache + pg * page_elems + (long)page_size * row + (long)e * page_size +
                                                  (key - pi * page_size));
      if (key + 8 > group_len) {                              // slots behind the last key may hold anything
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = key + j < group_len ? v[j] : (bf16_t)0.f;
      }
      return v;
    };
    auto k_store = [&](int i, const bf16x8& v) {
      const int kr = i / row8;
      if (i < 32 * row8) *reinterpret_cast<bf16x8*>(ks + kr * KLD + 8 * (i - kr * row8)) = v;
    };
    auto v_store = [&](int i, const bf16x8& v) {
      if (i >= rank * 4) return;
      bf16_t* dst = vs + (i / 4) * VLD + 8 * (i % 4);         // 8-byte aligned
      *reinterpret_cast<bf16x4*>(dst) = bf16x4{v[0], v[1], v[2], v[3]};
      *reinterpret_cast<bf16x4*>(dst + 4) = bf16x4{v[4], v[5], v[6], v[7]};
    };
    auto fetch = [&](int kb) -> Stage {
      Stage T;
#pragma unroll
      for (int j = 0; j < KP; ++j) T.k[j] = k_piece(tid + 64 * kLatWaves * j, kb);
#pragma unroll
      for (int j = 0; j < VP; ++j) T.v[j] = v_piece(tid + 64 * kLatWaves * j, kb);
      return T;
    };
    Stage st;
    if constexpr (KS > 0) st = fetch(0);
    for (int kb = 0; kb < group_len; kb += 32) {
      __syncthreads();                                        // the tile before this one has been read
      if constexpr (KS > 0) {
#pragma unroll
        for (int j = 0; j < KP; ++j) k_store(tid + 64 * kLatWaves * j, st.k[j]);
#pragma unroll
        for (int j = 0; j < VP; ++j) v_store(tid + 64 * kLatWaves * j, st.v[j]);
      } else {
        for (int i = tid; i < 32 * row8; i += 64 * kLatWaves) k_store(i, k_piece(i, kb));
        for (int i = tid; i < rank * 4; i += 64 * kLatWaves) v_store(i, v_piece(i, kb));
      }
      __syncthreads();
      if constexpr (KS > 0) {
        if (kb + 32 < group_len) st = fetch(kb + 32);         // (the same for all: no barrier inside)
      }
      if (!mine || kb >= len) continue;
      // ---- scores
      floatx4 s[2] = {floatx4{0.f, 0.f, 0.f, 0.f}, floatx4{0.f, 0.f, 0.f, 0.f}};
      auto score_step = [&](int kk, const bf16x8& qb) {
        const int d0 = 32 * kk + 8 * g;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const bf16x8 a = d0 < row ? *reinterpret_cast<const bf16x8*>(ks + (16 * u + c) * KLD + d0) : zero8;
          s[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qb, s[u], 0, 0, 0);
        }
      };
      if constexpr (KS > 0) {
#pragma unroll
        for (int kk = 0; kk < KS; ++kk)
          if (kk < ksteps) score_step(kk, qreg[kk]);
      } else {
        for (int kk = 0; kk < ksteps; ++kk) {
          const int d0 = 32 * kk + 8 * g;
          score_step(kk, (d0 < row && head_ok) ? *reinterpret_cast<const bf16x8*>(qrow + d0) : zero8);
        }
      }
      float tmax = -INFINITY;
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = kb + 16 * u + 4 * g + i;
          s[u][i] = key < len ? s[u][i] * scale : -INFINITY;
          tmax = fmaxf(tmax, s[u][i]);
        }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, kWave));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, kWave));
      const float m_new = fmaxf(m, tmax);                    // finite: kb < len
      const float alpha = expf(m - m_new);
      bf16x8 pb;
      float psum = 0.f;
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float p = (s[u][i] == -INFINITY) ? 0.f : expf(s[u][i] - m_new);
          const bf16_t pr = (bf16_t)p;
          pb[4 * u + i] = pr;
          psum += (float)pr;
        }
      l = l * alpha + psum;
      m = m_new;
      // ---- the weighted sum of the latents (keys beyond this token's last: probability 0, and
      // what LDS holds of them is another token's key or zero, never anything else)
#pragma unroll
      for (int r = 0; r < NR; ++r) {
        if (r < nr) {
          acc[r] *= alpha;
          const bf16_t* vrow = vs + (16 * r + c) * VLD + 4 * g;
          const bf16x4 lo = *reinterpret_cast<const bf16x4*>(vrow);
          const bf16x4 hi = *reinterpret_cast<const bf16x4*>(vrow + 16);
          const bf16x8 a = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
          acc[r] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb, acc[r], 0, 0, 0);
        }
      }
    }
    first = last + 1;
  }
  l += __shfl_xor(l, 16, kWave);
  l += __shfl_xor(l, 32, kWave);
  if (!token_ok || !head_ok) return;
  const float inv = 1.f / l;
  bf16_t* orow = out + ((long)t * H + head) * rank;
#pragma unroll
  for (int r = 0; r < NR; ++r) {
    if (r < nr) {
      bf16x4 v;
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = (bf16_t)(acc[r][i] * inv);
      *reinterpret_cast<bf16x4*>(orow + 16 * r + 4 * g) = v;
    }
  }
}

// The slices' results of one (token, head) become its output: weights exp(m_s - max m).
__global__ __launch_bounds__(kLatThreads) void attn_latent_merge_kernel(const float* __restrict__ part,
                                                                        bf16_t* __restrict__ out, int rank, int nslices) {
  const long th = blockIdx.x;
  const float* rows = part + th * nslices * (rank + 2);
  float M = -INFINITY;
  for (int s = 0; s < nslices; ++s) M = fmaxf(M, rows[(long)s * (rank + 2) + rank]);
  float l = 0.f;
  for (int s = 0; s < nslices; ++s) {
    const float ms = rows[(long)s * (rank + 2) + rank];
    if (ms != -INFINITY) l += expf(ms - M) * rows[(long)s * (rank + 2) + rank + 1];
  }
  const float inv = 1.f / l;
  for (int e = threadIdx.x; e < rank; e += kLatThreads) {
    float o = 0.f;
    for (int s = 0; s < nslices; ++s) {
      const float ms = rows[(long)s * (rank + 2) + rank];
      if (ms != -INFINITY) o = fmaf(expf(ms - M), rows[(long)s * (rank + 2) + e], o);
    }
    out[th * rank + e] = (bf16_t)(o * inv);
  }
}

template <int NR, int KS>
static void launch_latent_mfma(const void* q, void* out, const void* cache, const int* positions, const int* span_of_token,
                               const int* block_table, int max_pages, int page_size, int n, int H, int row, int rank,
                               float scale, float* part, int nslices, hipStream_t stream) {
  const size_t lds = (size_t)(kLatWaves - 1) * (NR * 4 + 2) * kWave * sizeof(float);
  const unsigned page_magic = (unsigned)(((1ull << 35) + page_size - 1) / page_size);
  static int raised = 0;
  if (lds > 64 * 1024 && !raised) {
    (void)hipFuncSetAttribute((const void*)attn_latent_mfma_kernel<NR, KS>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    raised = 1;
  }
  if (nslices == 0) {       // steps of many tokens: four tokens a workgroup, their keys through LDS
    const size_t tiles = ((size_t)32 * (row + 8) + (size_t)rank * 36) * sizeof(bf16_t);
    static size_t raised_to = 64 * 1024;
    if (tiles > raised_to) {
      (void)hipFuncSetAttribute((const void*)attn_latent_block_kernel<NR, KS>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)tiles);
      raised_to = tiles;
    }
    hipLaunchKernelGGL((attn_latent_block_kernel<NR, KS>), dim3((n + kLatWaves - 1) / kLatWaves, (H + 15) / 16), dim3(64 * kLatWaves),
                       tiles, stream, (const bf16_t*)q, (bf16_t*)out, (const bf16_t*)cache, positions, span_of_token,
                       block_table, max_pages, page_size, page_magic, n, H, row, rank, scale);
    return;
  }
  hipLaunchKernelGGL((attn_latent_mfma_kernel<NR, KS>), dim3(n, (H + 15) / 16, nslices), dim3(64 * kLatWaves), lds, stream,
                     (const bf16_t*)q, (bf16_t*)out, (const bf16_t*)cache, positions, span_of_token, block_table, max_pages,
                     page_size, page_magic, H, row, rank, scale, part);
  if (nslices > 1)
    hipLaunchKernelGGL(attn_latent_merge_kernel, dim3(n * H), dim3(kLatThreads), 0, stream, part, (bf16_t*)out, rank, nslices);
}

// attended: [n][H][rank]; w_uv [H * dv][rank]; gate: [nsplit][n][H * dv] sums or null.
template <typename T>
__global__ __launch_bounds__(kLatThreads) void latent_out_kernel(
    const T* __restrict__ attended, const T* __restrict__ w_uv, const float* __restrict__ gate, int nsplit,
    long split_stride, long gate_stride, T* __restrict__ out, int H, int dv, int rank) {
  extern __shared__ float al[];          // [rank]
  const long t = blockIdx.x;
  const int h = blockIdx.y, tid = threadIdx.x;
  const T* src = attended + (t * H + h) * rank;
  for (int i = tid; i < rank; i += kLatThreads) al[i] = to_f32(src[i]);
  __syncthreads();
  for (int j = tid; j < dv; j += kLatThreads) {
    const T* w = w_uv + ((long)h * dv + j) * rank;
    float acc = 0.f;
    for (int r = 0; r < rank; ++r) acc = fmaf(al[r], to_f32(w[r]), acc);
    const long col = (long)h * dv + j;
    if (gate) {
      float g = 0.f;
      for (int s = 0; s < nsplit; ++s) g += gate[s * split_stride + t * gate_stride + col];
      acc *= sigmoid_f32(g);
    }
    out[t * H * dv + col] = from_f32<T>(acc);
  }
}

// The two products with a head's own matrix on the matrix cores (bfloat16), MFMA 16x16x32 as
// above: a wave takes 16 outputs (rows of the head's matrix, one per lane, 16 bytes at a time)
// and 16 tokens, a workgroup four such pieces of 16 outputs.
//   latent_out:   out[t][h][j] = sum_r W_uv[h dv + j][r] attended[t][h][r], times the gate
//   latent_query: out[t][h][r] = sum_i W_ukT[h][r][i] q[t][h][i] (W_ukT: the head's matrix
//                 transposed once, when the weights are bound), and the rotated part beside it
__global__ __launch_bounds__(kLatThreads) void latent_out_mfma_kernel(
    const bf16_t* __restrict__ attended, const bf16_t* __restrict__ w_uv, const float* __restrict__ gate, int nsplit,
    long split_stride, long gate_stride, bf16_t* __restrict__ out, int n, int H, int dv, int rank) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int g = lane / 16, c = lane % 16;
  const int h = blockIdx.y;
  const int j0 = (blockIdx.z * 4 + wave) * 16;
  if (j0 >= dv) return;
  const int t = min((int)blockIdx.x * 16 + c, n - 1);
  const int j = min(j0 + c, dv - 1);
  const bf16_t* wrow = w_uv + ((long)h * dv + j) * rank;
  const bf16_t* arow = attended + ((long)t * H + h) * rank;
  floatx4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 8 * g; k0 < rank; k0 += 32) {            // rank % 32 == 0 (the launch): every lane takes every step
    const bf16x8 a = *reinterpret_cast<const bf16x8*>(wrow + k0);
    const bf16x8 b = *reinterpret_cast<const bf16x8*>(arow + k0);
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc, 0, 0, 0);
  }
  const int tt = blockIdx.x * 16 + c;
  if (tt >= n) return;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int jj = j0 + 4 * g + i;
    if (jj >= dv) continue;
    const long col = (long)h * dv + jj;
    float v = acc[i];
    if (gate) {
      float gs = 0.f;
      for (int s = 0; s < nsplit; ++s) gs += gate[s * split_stride + tt * gate_stride + col];
      v *= sigmoid_f32(gs);
    }
    out[(long)tt * H * dv + col] = (bf16_t)v;
  }
}

__global__ __launch_bounds__(kLatThreads) void latent_query_mfma_kernel(
    const float* __restrict__ q, int nsplit, long split_stride, const bf16_t* __restrict__ w_ukt,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, bf16_t* __restrict__ out, int n, int H, int d,
    int dr, int rank) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int g = lane / 16, c = lane % 16;
  const int h = blockIdx.y;
  const int hw = d + dr, half = dr / 2;
  const int t = min((int)blockIdx.x * 16 + c, n - 1);
  const int tt = blockIdx.x * 16 + c;
  const float* in = q + ((long)t * H + h) * hw;
  const int r0 = (blockIdx.z * 4 + wave) * 16;
  if (r0 < rank) {
    const int r = min(r0 + c, rank - 1);
    const bf16_t* wrow = w_ukt + ((long)h * rank + r) * d;
    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int k0 = 8 * g; k0 < d; k0 += 32) {               // d % 32 == 0 (the launch)
      const bf16x8 a = *reinterpret_cast<const bf16x8*>(wrow + k0);
      bf16x8 b;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float v = 0.f;
        for (int s = 0; s < nsplit; ++s) v += in[s * split_stride + k0 + e];
        b[e] = (bf16_t)v;
      }
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc, 0, 0, 0);
    }
    if (tt < n) {
      bf16_t* dst = out + ((long)tt * H + h) * (rank + dr);
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (r0 + 4 * g + i < rank) dst[r0 + 4 * g + i] = (bf16_t)acc[i];
    }
  }
  // the rotated part: the workgroup's first piece of outputs takes it along
  if (blockIdx.z == 0 && wave == 0 && tt < n) {
    bf16_t* dst = out + ((long)tt * H + h) * (rank + dr);
    for (int i = g; i < half; i += 4) {
      float a = 0.f, b = 0.f;
      for (int s = 0; s < nsplit; ++s) {
        a += in[s * split_stride + d + i];
        b += in[s * split_stride + d + half + i];
      }
      const float cs = cos_t[(long)tt * half + i], sn = sin_t[(long)tt * half + i];
      dst[rank + i] = (bf16_t)(a * cs - b * sn);
      dst[rank + half + i] = (bf16_t)(b * cs + a * sn);
    }
  }
}

}  // namespace kllm

using namespace kllm;

extern "C" int kllm_latent_max_row(void) { return kLatMaxRow; }

extern "C" int kllm_latent_kv_append(const float* dkv, int nsplit, long split_stride, const float* weight, float eps,
                                     const float* cos_t, const float* sin_t, void* cache, const int* positions,
                                     const int* span_of_token, const int* block_table, int max_pages, int page_size,
                                     int n, int rank, int dr, int dtype, long in_stride, hipStream_t stream) {
  KLLM_REQUIRE(dkv && weight && cos_t && sin_t && cache && positions && span_of_token && block_table,
               "latent_kv_append: null pointer");
  KLLM_REQUIRE(n > 0 && nsplit >= 1 && rank > 0 && dr > 0 && dr % 2 == 0 && rank + dr <= kLatMaxRow,
               "latent_kv_append: bad sizes n=%d rank=%d dr=%d (rows of up to %d)", n, rank, dr, kLatMaxRow);
  KLLM_REQUIRE(max_pages > 0 && page_size > 0, "latent_kv_append: bad cache sizes");
  KLLM_REQUIRE(dtype == DT_F32 || dtype == DT_BF16, "latent_kv_append: unknown dtype %d", dtype);
  if (dtype == DT_F32)
    hipLaunchKernelGGL(latent_kv_append_kernel<float>, dim3(n), dim3(kLatThreads), 0, stream, dkv, nsplit, split_stride,
                       weight, eps, cos_t, sin_t, (float*)cache, positions, span_of_token, block_table, max_pages,
                       page_size, rank, dr, in_stride);
  else
    hipLaunchKernelGGL(latent_kv_append_kernel<bf16_t>, dim3(n), dim3(kLatThreads), 0, stream, dkv, nsplit,
                       split_stride, weight, eps, cos_t, sin_t, (bf16_t*)cache, positions, span_of_token, block_table,
                       max_pages, page_size, rank, dr, in_stride);
  KLLM_CHECK_LAUNCH("latent_kv_append");
  return 0;
}

extern "C" int kllm_latent_norm(const float* in, int nsplit, long split_stride, long in_stride, const float* weight,
                                float eps, void* out, int n, int r, int dtype, hipStream_t stream) {
  KLLM_REQUIRE(in && weight && out && n > 0 && r > 0 && nsplit >= 1 && in_stride >= r, "latent_norm: null pointer or bad sizes");
  KLLM_REQUIRE(dtype == DT_F32 || dtype == DT_BF16, "latent_norm: unknown dtype %d", dtype);
  if (dtype == DT_F32)
    hipLaunchKernelGGL(latent_norm_kernel<float>, dim3(n), dim3(kLatThreads), 0, stream, in, nsplit, split_stride,
                       in_stride, weight, eps, (float*)out, r);
  else
    hipLaunchKernelGGL(latent_norm_kernel<bf16_t>, dim3(n), dim3(kLatThreads), 0, stream, in, nsplit, split_stride,
                       in_stride, weight, eps, (bf16_t*)out, r);
  KLLM_CHECK_LAUNCH("latent_norm");
  return 0;
}

extern "C" int kllm_latent_query(const float* q, int nsplit, long split_stride, const void* w_uk, const float* cos_t,
                                 const float* sin_t, void* out, int n, int H, int d, int dr, int rank, int dtype,
                                 int transposed, hipStream_t stream) {
  KLLM_REQUIRE(q && w_uk && cos_t && sin_t && out, "latent_query: null pointer");
  KLLM_REQUIRE(n > 0 && nsplit >= 1 && H > 0 && H <= 65535 && d > 0 && dr > 0 && dr % 2 == 0 && rank > 0 &&
                   rank + dr <= kLatMaxRow && d + dr <= 4096,
               "latent_query: bad sizes n=%d H=%d d=%d dr=%d rank=%d", n, H, d, dr, rank);
  KLLM_REQUIRE(dtype == DT_F32 || dtype == DT_BF16, "latent_query: unknown dtype %d", dtype);
  if (transposed) {     // w_uk is [H][rank][d]: the kernel on the matrix cores
    KLLM_REQUIRE(dtype == DT_BF16 && d % 32 == 0 && ((uintptr_t)w_uk & 15) == 0,
                 "latent_query: the transposed matrix goes with bfloat16 and head sizes in steps of 32 (d=%d)", d);
    hipLaunchKernelGGL(latent_query_mfma_kernel, dim3((n + 15) / 16, H, (rank + 63) / 64), dim3(kLatThreads), 0, stream, q,
                       nsplit, split_stride, (const bf16_t*)w_uk, cos_t, sin_t, (bf16_t*)out, n, H, d, dr, rank);
    KLLM_CHECK_LAUNCH("latent_query");
    return 0;
  }
  const size_t lds = (size_t)(d + dr) * sizeof(float);
  if (dtype == DT_F32)
    hipLaunchKernelGGL(latent_query_kernel<float>, dim3(n, H), dim3(kLatThreads), lds, stream, q, nsplit, split_stride,
                       (const float*)w_uk, cos_t, sin_t, (float*)out, H, d, dr, rank);
  else
    hipLaunchKernelGGL(latent_query_kernel<bf16_t>, dim3(n, H), dim3(kLatThreads), lds, stream, q, nsplit, split_stride,
                       (const bf16_t*)w_uk, cos_t, sin_t, (bf16_t*)out, H, d, dr, rank);
  KLLM_CHECK_LAUNCH("latent_query");
  return 0;
}

extern "C" int kllm_attn_latent(const void* q, void* out, const void* cache, const int* positions,
                                const int* span_of_token, const int* block_table, int max_pages, int page_size, int n,
                                int H, int row, int rank, float scale, int dtype, int mode, float* part, long part_floats, int nslices,
                                hipStream_t stream) {
  KLLM_REQUIRE(q && out && cache && positions && span_of_token && block_table, "attn_latent: null pointer");
  KLLM_REQUIRE(n > 0 && H > 0 && H <= 65535 && rank > 0 && rank <= row && row <= kLatMaxRow,
               "attn_latent: bad sizes n=%d H=%d row=%d rank=%d (rows of up to %d)", n, H, row, rank, kLatMaxRow);
  KLLM_REQUIRE(max_pages > 0 && page_size > 0, "attn_latent: bad cache sizes");
  KLLM_REQUIRE(dtype == DT_F32 || dtype == DT_BF16, "attn_latent: unknown dtype %d", dtype);
  if (dtype == DT_BF16 && mode != 1 && rank % 16 == 0 && row % 8 == 0 && rank <= 512 && page_size % 16 == 0 &&
      page_size <= 2048 && (long)max_pages * page_size <= (1L << 24) &&
      ((uintptr_t)q & 15) == 0 && ((uintptr_t)cache & 15) == 0 && ((uintptr_t)out & 7) == 0) {
    KLLM_REQUIRE(nslices >= 0 && nslices <= 64 && (nslices <= 1 || (part && part_floats >= (long)n * H * nslices * (rank + 2))),
                 "attn_latent: %d slices need room for %d tokens x %d heads x %d slices x (%d + 2) floats", nslices, n, H,
                 nslices, rank);
    // the latent's accumulators and the query's pieces in registers: built for ranks up to 128, 256 and
    // 512 with rows of up to 256, 384 and 640; longer rows ask for the query at every tile
#define KLLM_LAT(NR, KS) launch_latent_mfma<NR, KS>(q, out, cache, positions, span_of_token, block_table, max_pages, page_size, n, H, row, rank, scale, part, nslices, stream)
    if (rank <= 128) { if (row <= 256) KLLM_LAT(8, 8); else KLLM_LAT(8, 0); }
    else if (rank <= 256) { if (row <= 384) KLLM_LAT(16, 12); else KLLM_LAT(16, 0); }
    else { if (row <= 640) KLLM_LAT(32, 20); else KLLM_LAT(32, 0); }
#undef KLLM_LAT
    KLLM_CHECK_LAUNCH("attn_latent");
    return 0;
  }
  if (dtype == DT_F32)
    hipLaunchKernelGGL(attn_latent_kernel<float>, dim3(n, H), dim3(kLatThreads), 0, stream, (const float*)q,
                       (float*)out, (const float*)cache, positions, span_of_token, block_table, max_pages, page_size, H,
                       row, rank, scale);
  else
    hipLaunchKernelGGL(attn_latent_kernel<bf16_t>, dim3(n, H), dim3(kLatThreads), 0, stream, (const bf16_t*)q,
                       (bf16_t*)out, (const bf16_t*)cache, positions, span_of_token, block_table, max_pages, page_size,
                       H, row, rank, scale);
  KLLM_CHECK_LAUNCH("attn_latent");
  return 0;
}

extern "C" int kllm_latent_out(const void* attended, const void* w_uv, const float* gate, int nsplit, long split_stride,
                               long gate_stride, void* out, int n, int H, int dv, int rank, int dtype,
                               hipStream_t stream) {
  KLLM_REQUIRE(attended && w_uv && out, "latent_out: null pointer");
  KLLM_REQUIRE(n > 0 && H > 0 && H <= 65535 && dv > 0 && rank > 0 && rank <= 8192 && (!gate || nsplit >= 1),
               "latent_out: bad sizes n=%d H=%d dv=%d rank=%d", n, H, dv, rank);
  KLLM_REQUIRE(dtype == DT_F32 || dtype == DT_BF16, "latent_out: unknown dtype %d", dtype);
  if (dtype == DT_BF16 && rank % 32 == 0 && ((uintptr_t)attended & 15) == 0 && ((uintptr_t)w_uv & 15) == 0) {
    hipLaunchKernelGGL(latent_out_mfma_kernel, dim3((n + 15) / 16, H, (dv + 63) / 64), dim3(kLatThreads), 0, stream,
                       (const bf16_t*)attended, (const bf16_t*)w_uv, gate, nsplit, split_stride, gate_stride, (bf16_t*)out,
                       n, H, dv, rank);
    KLLM_CHECK_LAUNCH("latent_out");
    return 0;
  }
  const size_t lds = (size_t)rank * sizeof(float);
  if (dtype == DT_F32)
    hipLaunchKernelGGL(latent_out_kernel<float>, dim3(n, H), dim3(kLatThreads), lds, stream, (const float*)attended,
                       (const float*)w_uv, gate, nsplit, split_stride, gate_stride, (float*)out, H, dv, rank);
  else
    hipLaunchKernelGGL(latent_out_kernel<bf16_t>, dim3(n, H), dim3(kLatThreads), lds, stream, (const bf16_t*)attended,
                       (const bf16_t*)w_uv, gate, nsplit, split_stride, gate_stride, (bf16_t*)out, H, dv, rank);
  KLLM_CHECK_LAUNCH("latent_out");
  return 0;
}
