// Per-token steps of layers whose norm stands behind the sub-layer instead of in front of it,
// and of attention whose queries and keys are normalised after their rotation:
//
//   kllm_norm_residual     x += m * w * N(d + b), or x = w * N(x); N(v) = v / sqrt(mean(v^2) + eps);
//                          optionally x rounded to the compute dtype for the next product, or
//                          N(x) times the weight of the norm in front of the next sub-layer
//   kllm_rope_tables_freq  cos/sin tables from a table of angles per position (any schedule of
//                          frequencies), times a constant factor
//   kllm_qkv_norm_append   biases, rotation of the leading elements of every head, unit RMS of
//                          every query and key head, queries out, keys and values into pages
//   kllm_gate_bias         the gate of a gated feed-forward whose two products have biases, or
//                          whose gate is clamped
//
// Everything here is computed in 32-bit; a row's result depends on the row alone.
#include <math.h>

#include "common.hpp"
#include "kllm_kernels.h"

namespace kllm {

constexpr int kRowThreads = 256;

// One workgroup per row.  PER > 0: a thread keeps its PER elements of the row in registers, and
// everything it reads (the sums' slices, the bias, the stream, the weight) is asked for before
// the first use, so that a row costs one trip to memory (decode batches: one row, one workgroup).
// PER == 0: rows of any length, the row's sums kept in LDS between the two passes.
// The sums may also be those of a token's chosen experts, not yet added up (`chosen`): then
// v = sum over the token's choices of wgt * (expert < E ? y[choice] : the feed-forward's input)
// + the slices of delta (a shared expert's) + the bias.
struct ChosenSums {
  const float* y;        // [n * top][d], null: none
  const void* xin;       // [n][d] in xin_dtype: what an identity expert hands on
  const int* idx;        // [n][top]
  const float* wgt;      // [n][top]
  int top, E, xin_dtype;
};

// Two sub-layers side by side whose outputs are each normed before they are added: the row is
// sa * wa * N(delta's slices) + sb * wb * N(b's slices) in place of delta's slices.
struct NormedPair {
  const float* b;        // [nb][n][d], null: no such pair
  const float* wa;       // [d]
  const float* wb;       // [d]
  long stride_b;
  int nb;
  float sa, sb;
};

template <typename TOUT, int PER>
__global__ __launch_bounds__(kRowThreads) void norm_residual_kernel(
    float* __restrict__ x, const float* __restrict__ delta, int nsplit, long split_stride,
    const float* __restrict__ bias, const float* __restrict__ w, TOUT* __restrict__ out, int d, float eps,
    const ChosenSums chosen, float mult, const float* __restrict__ next_w, const float* __restrict__ delta_scale,
    const NormedPair pair) {
  extern __shared__ float row_lds[];      // [d] (PER == 0; twice that with a pair)
  __shared__ float red[16];
  const long r = blockIdx.x;
  const float dscale = delta_scale ? delta_scale[r] : 1.f;      // a factor of the row's delta (a gate of a shared expert)
  float* xr = x + r * d;
  const bool sums = delta || chosen.y;    // otherwise the stream itself is normalised
  auto chosen_at = [&](int i) {
    float t = 0.f;
    for (int s = 0; s < chosen.top; ++s) {
      const long entry = r * chosen.top + s;
      float part;
      if (chosen.idx[entry] < chosen.E)
        part = chosen.y[entry * d + i];
      else
        part = chosen.xin_dtype == DT_BF16 ? to_f32(reinterpret_cast<const bf16_t*>(chosen.xin)[r * d + i])
                                           : reinterpret_cast<const float*>(chosen.xin)[r * d + i];
      t = fmaf(chosen.wgt[entry], part, t);
    }
    return t;
  };
  if constexpr (PER > 0) {
    // Loops over slices and choices stand outside the loop over a thread's elements, whose
    // loads then go out together (a load behind a loop of unknown length is waited for at once).
    float v[PER], xv[PER], wv[PER];
    int at[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int i = threadIdx.x + kRowThreads * j;
      at[j] = i < d ? i : 0;
      xv[j] = xr[at[j]];
      wv[j] = w[at[j]];
      v[j] = 0.f;
    }
    if (sums) {
      if (chosen.y) {
        for (int s = 0; s < chosen.top; ++s) {
          const long entry = r * chosen.top + s;
          const float weight = chosen.wgt[entry];
          if (chosen.idx[entry] < chosen.E) {
            const float* src = chosen.y + entry * d;
#pragma unroll
            for (int j = 0; j < PER; ++j) v[j] = fmaf(weight, src[at[j]], v[j]);
          } else if (chosen.xin_dtype == DT_BF16) {
            const bf16_t* src = reinterpret_cast<const bf16_t*>(chosen.xin) + r * d;
#pragma unroll
            for (int j = 0; j < PER; ++j) v[j] = fmaf(weight, to_f32(src[at[j]]), v[j]);
          } else {
            const float* src = reinterpret_cast<const float*>(chosen.xin) + r * d;
#pragma unroll
            for (int j = 0; j < PER; ++j) v[j] = fmaf(weight, src[at[j]], v[j]);
          }
        }
      }
      if (delta) {
        float dv[PER];
#pragma unroll
        for (int j = 0; j < PER; ++j) dv[j] = 0.f;
        for (int s = 0; s < nsplit; ++s) {
          const float* src = delta + s * split_stride + r * d;
#pragma unroll
          for (int j = 0; j < PER; ++j) dv[j] += src[at[j]];
        }
        if (pair.b) {       // each of the two normed over the row before they are added
          float bv[PER], wa[PER], wb[PER];
#pragma unroll
          for (int j = 0; j < PER; ++j) {
            bv[j] = 0.f;
            wa[j] = pair.wa[at[j]];
            wb[j] = pair.wb[at[j]];
          }
          for (int s = 0; s < pair.nb; ++s) {
            const float* src = pair.b + s * pair.stride_b + r * d;
#pragma unroll
            for (int j = 0; j < PER; ++j) bv[j] += src[at[j]];
          }
          float ssa = 0.f, ssb = 0.f;
#pragma unroll
          for (int j = 0; j < PER; ++j) {
            if (threadIdx.x + kRowThreads * j >= d) dv[j] = bv[j] = 0.f;
            ssa = fmaf(dv[j], dv[j], ssa);
            ssb = fmaf(bv[j], bv[j], ssb);
          }
          const float ra = pair.sa / sqrtf(block_sum(ssa, red) / (float)d + eps);
          const float rb = pair.sb / sqrtf(block_sum(ssb, red) / (float)d + eps);
#pragma unroll
          for (int j = 0; j < PER; ++j) dv[j] = fmaf(dv[j] * ra, wa[j], bv[j] * rb * wb[j]);
        }
#pragma unroll
        for (int j = 0; j < PER; ++j) v[j] = fmaf(dscale, dv[j], v[j]);
      }
      if (bias) {
#pragma unroll
        for (int j = 0; j < PER; ++j) v[j] += bias[at[j]];
      }
    } else {
#pragma unroll
      for (int j = 0; j < PER; ++j) v[j] = xv[j];
    }
#pragma unroll
    for (int j = 0; j < PER; ++j)
      if (threadIdx.x + kRowThreads * j >= d) v[j] = 0.f;
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < PER; ++j) ss = fmaf(v[j], v[j], ss);
    const float rstd = 1.f / sqrtf(block_sum(ss, red) / (float)d + eps);
    float ss2 = 0.f;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int i = threadIdx.x + kRowThreads * j;
      const float y = v[j] * rstd * wv[j];
      v[j] = i < d ? (sums ? fmaf(mult, y, xv[j]) : y) : 0.f;
      if (i < d) xr[i] = v[j];
      ss2 = fmaf(v[j], v[j], ss2);
    }
    if (!out) return;
    if (next_w) {       // the norm in front of the next sub-layer, of the row that is still in registers
#pragma unroll
      for (int j = 0; j < PER; ++j) wv[j] = next_w[at[j]];
      const float rstd2 = 1.f / sqrtf(block_sum(ss2, red) / (float)d + eps);
#pragma unroll
      for (int j = 0; j < PER; ++j) v[j] = v[j] * rstd2 * wv[j];
    }
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int i = threadIdx.x + kRowThreads * j;
      if (i < d) out[r * d + i] = from_f32<TOUT>(v[j]);
    }
    return;
  }
  float ra = 1.f, rb = 0.f;
  if (pair.b) {       // a pass of its own for the two sums of squares; the sums wait in LDS
    float ssa = 0.f, ssb = 0.f;
    for (int i = threadIdx.x; i < d; i += kRowThreads) {
      float a = 0.f, b = 0.f;
      for (int s = 0; s < nsplit; ++s) a += delta[s * split_stride + r * d + i];
      for (int s = 0; s < pair.nb; ++s) b += pair.b[s * pair.stride_b + r * d + i];
      row_lds[i] = a;
      row_lds[d + i] = b;
      ssa = fmaf(a, a, ssa);
      ssb = fmaf(b, b, ssb);
    }
    ra = pair.sa / sqrtf(block_sum(ssa, red) / (float)d + eps);
    rb = pair.sb / sqrtf(block_sum(ssb, red) / (float)d + eps);
  }
  float ss = 0.f;
  for (int i = threadIdx.x; i < d; i += kRowThreads) {
    float v;
    if (sums) {
      v = chosen.y ? chosen_at(i) : 0.f;
      if (pair.b) {
        v = fmaf(dscale, fmaf(row_lds[i] * ra, pair.wa[i], row_lds[d + i] * rb * pair.wb[i]), v);
      } else if (delta) {
        float dsum = 0.f;
        for (int s = 0; s < nsplit; ++s) dsum += delta[s * split_stride + r * d + i];
        v = fmaf(dscale, dsum, v);
      }
      if (bias) v += bias[i];
    } else {
      v = xr[i];
    }
    row_lds[i] = v;
    ss = fmaf(v, v, ss);
  }
  const float total = block_sum(ss, red);
  const float rstd = 1.f / sqrtf(total / (float)d + eps);
  float ss2 = 0.f;
  for (int i = threadIdx.x; i < d; i += kRowThreads) {    // a thread reads back what it wrote itself
    const float y = row_lds[i] * rstd * w[i];
    const float v = sums ? fmaf(mult, y, xr[i]) : y;
    xr[i] = v;
    row_lds[i] = v;
    ss2 = fmaf(v, v, ss2);
    if (out && !next_w) out[r * d + i] = from_f32<TOUT>(v);
  }
  if (!out || !next_w) return;
  const float rstd2 = 1.f / sqrtf(block_sum(ss2, red) / (float)d + eps);
  for (int i = threadIdx.x; i < d; i += kRowThreads) out[r * d + i] = from_f32<TOUT>(row_lds[i] * rstd2 * next_w[i]);
}

__global__ void rope_tables_freq_kernel(float* __restrict__ cos_t, float* __restrict__ sin_t,
                                        const int* __restrict__ positions, const double* __restrict__ freq, int n,
                                        int half, double factor) {
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long)n * half) return;
  const int t = (int)(idx / half), i = (int)(idx % half);
  double sn, cs;
  sincos((double)positions[t] * freq[i], &sn, &cs);
  cos_t[idx] = (float)(cs * factor);
  sin_t[idx] = (float)(sn * factor);
}

// One wave per (token, item): the items of a token are its H query heads, its KV key heads and
// its KV value heads.  A lane holds up to two pairs of a head of up to 256.
template <typename T>
__global__ __launch_bounds__(256) void qkv_norm_append_kernel(
    const float* __restrict__ qkv, int nsplit, long split_stride, const float* __restrict__ bias,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rot, int interleaved, int unit_norm,
    float eps, T* __restrict__ q_out, T* __restrict__ cache, const int* __restrict__ positions,
    const int* __restrict__ span_of_token, const int* __restrict__ block_table, int max_pages, int page_size,
    int H, int KV, int dk, int dv, const float* __restrict__ q_weight, const float* __restrict__ k_weight) {
  const long t = blockIdx.x;
  const int lane = threadIdx.x % kWave;
  const int item = blockIdx.y * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (item >= H + 2 * KV) return;
  const long cols = (long)(H + KV) * dk + (long)KV * dv;
  const float* in = qkv + t * cols;
  const int pos = positions[t];
  const long page = block_table[(long)span_of_token[t] * max_pages + pos / page_size];
  const int slot = pos % page_size;
  const long kblock = (long)page_size * dk, vblock = (long)page_size * dv;
  T* page_base = cache + page * KV * (kblock + vblock);
  // Loops over the sums' slices stand outside the loops over a lane's elements, whose loads then
  // go out together.
  if (item >= H + KV) {     // a value head: stored with the slot as the fast index
    const int h = item - H - KV;
    const long vcol = (long)(H + KV) * dk + h * dv;
    float v[4];
    int col[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int j = lane + kWave * r;
      col[r] = j < dv ? j : 0;
      v[r] = 0.f;
    }
    for (int s = 0; s < nsplit; ++s) {
      const float* src = in + s * split_stride + vcol;
#pragma unroll
      for (int r = 0; r < 4; ++r) v[r] += src[col[r]];
    }
    T* vdst = page_base + KV * kblock + h * vblock + slot;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int j = lane + kWave * r;
      if (j < dv) vdst[(long)j * page_size] = from_f32<T>(bias ? v[r] + bias[vcol + j] : v[r]);
    }
    return;
  }
  const bool is_q = item < H;
  const int h = is_q ? item : item - H;
  const long base = (long)item * dk;         // queries first, then keys, head after head
  const int pairs = dk / 2, rhalf = rot / 2;
  float ra[2], rb[2];
  int ea[2], eb[2];
  float a[2] = {0.f, 0.f}, b[2] = {0.f, 0.f};
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    const int j = lane + kWave * r;
    // the two elements of this pair: one that turns, or two neighbours that pass through
    ea[r] = j >= pairs ? 0 : j < rhalf ? (interleaved ? 2 * j : j) : rot + 2 * (j - rhalf);
    eb[r] = j >= pairs ? 0 : j < rhalf ? (interleaved ? 2 * j + 1 : j + rhalf) : ea[r] + 1;
  }
  for (int s = 0; s < nsplit; ++s) {
    const float* src = in + s * split_stride + base;
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      a[r] += src[ea[r]];
      b[r] += src[eb[r]];
    }
  }
  if (bias) {
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      if (lane + kWave * r >= pairs) continue;
      a[r] += bias[base + ea[r]];
      b[r] += bias[base + eb[r]];
    }
  }
  const float* nw = is_q ? q_weight : k_weight;
  if (nw) {     // a norm with weights in front of the rotation
    float s0 = 0.f;
#pragma unroll
    for (int r = 0; r < 2; ++r)
      if (lane + kWave * r < pairs) s0 += a[r] * a[r] + b[r] * b[r];
    const float rs = 1.f / sqrtf(wave_sum(s0) / (float)dk + eps);
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      if (lane + kWave * r >= pairs) continue;
      a[r] = a[r] * rs * nw[ea[r]];
      b[r] = b[r] * rs * nw[eb[r]];
    }
    unit_norm = 0;
  }
  float ss = 0.f;
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    const int j = lane + kWave * r;
    ra[r] = rb[r] = 0.f;
    if (j >= pairs) continue;
    const bool turns = cos_t && j < rhalf;
    const float c = turns ? cos_t[t * rhalf + j] : 1.f, sn = turns ? sin_t[t * rhalf + j] : 0.f;
    ra[r] = a[r] * c - b[r] * sn;
    rb[r] = b[r] * c + a[r] * sn;
    ss += ra[r] * ra[r] + rb[r] * rb[r];
  }
  float rstd = 1.f;
  if (unit_norm) rstd = 1.f / sqrtf(wave_sum(ss) / (float)dk + eps);
  T* dst = is_q ? q_out + (t * H + h) * dk : page_base + h * kblock + (long)slot * dk;
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    if (lane + kWave * r >= pairs) continue;
    dst[ea[r]] = from_f32<T>(ra[r] * rstd);
    dst[eb[r]] = from_f32<T>(rb[r] * rstd);
  }
}

template <typename TOUT>
__global__ void gate_bias_kernel(const float* __restrict__ gu, int nsplit, long split_stride,
                                 const float* __restrict__ bias, TOUT* __restrict__ out, long count, int f, int act,
                                 float limit, float alpha) {
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= count) return;
  const long t = idx / f;
  const int j = (int)(idx % f);
  const float* row = gu + t * 2 * f;
  float g = 0.f, u = 0.f;
  for (int s = 0; s < nsplit; ++s) {
    g += row[s * split_stride + j];
    u += row[s * split_stride + f + j];
  }
  if (bias) {
    g += bias[j];
    u += bias[f + j];
  }
  out[idx] = from_f32<TOUT>(gated(g, u, act, limit, alpha));
}

}  // namespace kllm

using namespace kllm;

extern "C" int kllm_norm_residual(float* x, const float* delta, int nsplit, long split_stride, const float* bias,
                                  const float* weight, void* out, int out_dtype, int n, int d, float eps,
                                  const float* chosen_y, const void* chosen_x, int chosen_x_dtype, const int* chosen_idx,
                                  const float* chosen_wgt, int top, int E, float mult, const float* next_weight,
                                  const float* delta_scale, const float* pair_b, int pair_nb, long pair_stride,
                                  const float* pair_wa, const float* pair_wb, float pair_sa, float pair_sb,
                                  hipStream_t stream) {
  KLLM_REQUIRE(x && weight, "norm_residual: null pointer");
  KLLM_REQUIRE(!pair_b || (delta && pair_wa && pair_wb && pair_nb >= 1 && !chosen_y),
               "norm_residual: two normed sums come with both sums and both weights, and without chosen experts");
  NormedPair pair;
  pair.b = pair_b; pair.wa = pair_wa; pair.wb = pair_wb; pair.stride_b = pair_stride; pair.nb = pair_nb;
  pair.sa = pair_sa; pair.sb = pair_sb;
  KLLM_REQUIRE(!next_weight || out, "norm_residual: the next norm's rows need a place");
  KLLM_REQUIRE(!delta_scale || delta, "norm_residual: a factor per row goes with sums");
  KLLM_REQUIRE(!chosen_y || (chosen_x && chosen_idx && chosen_wgt && top > 0 && E >= 0 &&
                             (chosen_x_dtype == DT_F32 || chosen_x_dtype == DT_BF16)),
               "norm_residual: the chosen experts' sums come with their input, choices and weights");
  ChosenSums chosen;
  chosen.y = chosen_y; chosen.xin = chosen_x; chosen.idx = chosen_idx; chosen.wgt = chosen_wgt;
  chosen.top = top; chosen.E = E; chosen.xin_dtype = chosen_x_dtype;
  KLLM_REQUIRE(n > 0 && d > 0 && d <= 16384, "norm_residual: bad sizes n=%d d=%d (rows of up to 16384)", n, d);
  KLLM_REQUIRE(!delta || nsplit >= 1, "norm_residual: nsplit %d", nsplit);
  KLLM_REQUIRE(delta || chosen_y || !bias, "norm_residual: a bias goes with sums");
  KLLM_REQUIRE(out_dtype == DT_F32 || out_dtype == DT_BF16, "norm_residual: unknown dtype %d", out_dtype);
#define KLLM_NR(TOUT, PER)                                                                                    \
  hipLaunchKernelGGL((norm_residual_kernel<TOUT, PER>), dim3(n), dim3(kRowThreads),                           \
                     PER ? 0 : (size_t)d * sizeof(float) * (pair_b ? 2 : 1), stream, x, delta, nsplit, split_stride, \
                     bias, weight, (TOUT*)out, d, eps, chosen, mult, next_weight, delta_scale, pair)
  const bool bf = out && out_dtype == DT_BF16;
  if (d <= 4 * kRowThreads) {
    if (bf) KLLM_NR(bf16_t, 4); else KLLM_NR(float, 4);
  } else if (d <= 8 * kRowThreads) {
    if (bf) KLLM_NR(bf16_t, 8); else KLLM_NR(float, 8);
  } else if (d <= 16 * kRowThreads) {
    if (bf) KLLM_NR(bf16_t, 16); else KLLM_NR(float, 16);
  } else {
    if (bf) KLLM_NR(bf16_t, 0); else KLLM_NR(float, 0);
  }
#undef KLLM_NR
  KLLM_CHECK_LAUNCH("norm_residual");
  return 0;
}

extern "C" int kllm_rope_tables_freq(float* cos_t, float* sin_t, const int* positions, const double* freq, int n,
                                     int half, double factor, hipStream_t stream) {
  KLLM_REQUIRE(cos_t && sin_t && positions && freq, "rope_tables_freq: null pointer");
  KLLM_REQUIRE(n > 0 && half > 0, "rope_tables_freq: bad sizes n=%d half=%d", n, half);
  hipLaunchKernelGGL(rope_tables_freq_kernel, dim3(ceil_div((long)n * half, 256)), dim3(256), 0, stream, cos_t, sin_t,
                     positions, freq, n, half, factor);
  KLLM_CHECK_LAUNCH("rope_tables_freq");
  return 0;
}

extern "C" int kllm_qkv_norm_append(const float* qkv, int nsplit, long split_stride, const float* bias,
                                    const float* cos_t, const float* sin_t, int rot, int interleaved, int unit_norm,
                                    float eps, void* q_out, void* cache, const int* positions,
                                    const int* span_of_token, const int* block_table, int max_pages, int page_size,
                                    int n, int H, int KV, int dk, int dv, int dtype, const float* q_weight,
                                    const float* k_weight, hipStream_t stream) {
  KLLM_REQUIRE(qkv && q_out && cache && positions && span_of_token && block_table, "qkv_norm_append: null pointer");
  KLLM_REQUIRE((q_weight == nullptr) == (k_weight == nullptr), "qkv_norm_append: the two norm weights go together");
  KLLM_REQUIRE(n > 0 && H > 0 && KV > 0 && nsplit >= 1, "qkv_norm_append: bad sizes n=%d H=%d KV=%d nsplit=%d", n, H, KV,
               nsplit);
  KLLM_REQUIRE(dk > 0 && dk % 2 == 0 && dk <= 256 && dv > 0 && dv <= 256,
               "qkv_norm_append: heads of %d (even) and values of %d, up to 256", dk, dv);
  KLLM_REQUIRE(rot >= 0 && rot <= dk && rot % 2 == 0 && (interleaved == 0 || interleaved == 1),
               "qkv_norm_append: rotary dimension %d of a head of %d", rot, dk);
  KLLM_REQUIRE((cos_t == nullptr) == (sin_t == nullptr), "qkv_norm_append: cos and sin go together");
  KLLM_REQUIRE(max_pages > 0 && page_size > 0, "qkv_norm_append: bad cache sizes");
  KLLM_REQUIRE(dtype == DT_F32 || dtype == DT_BF16, "qkv_norm_append: unknown dtype %d", dtype);
  const dim3 grid(n, ceil_div(H + 2 * KV, 4));
  if (dtype == DT_F32)
    hipLaunchKernelGGL(qkv_norm_append_kernel<float>, grid, dim3(256), 0, stream, qkv, nsplit, split_stride, bias, cos_t,
                       sin_t, rot, interleaved, unit_norm, eps, (float*)q_out, (float*)cache, positions, span_of_token,
                       block_table, max_pages, page_size, H, KV, dk, dv, q_weight, k_weight);
  else
    hipLaunchKernelGGL(qkv_norm_append_kernel<bf16_t>, grid, dim3(256), 0, stream, qkv, nsplit, split_stride, bias, cos_t,
                       sin_t, rot, interleaved, unit_norm, eps, (bf16_t*)q_out, (bf16_t*)cache, positions, span_of_token,
                       block_table, max_pages, page_size, H, KV, dk, dv, q_weight, k_weight);
  KLLM_CHECK_LAUNCH("qkv_norm_append");
  return 0;
}

extern "C" int kllm_gate_bias(const float* gu, int nsplit, long split_stride, const float* bias, void* out,
                              int out_dtype, int n, int f, int act, float limit, float alpha, hipStream_t stream) {
  KLLM_REQUIRE(gu && out, "gate_bias: null pointer");
  KLLM_REQUIRE(n > 0 && f > 0 && nsplit >= 1, "gate_bias: bad sizes n=%d f=%d nsplit=%d", n, f, nsplit);
  KLLM_REQUIRE(gated_known(act), "gate_bias: unknown activation %d", act);
  KLLM_REQUIRE(out_dtype == DT_F32 || out_dtype == DT_BF16, "gate_bias: unknown dtype %d", out_dtype);
  const long count = (long)n * f;
  const dim3 grid(ceil_div(count, 256));
  if (out_dtype == DT_BF16)
    hipLaunchKernelGGL(gate_bias_kernel<bf16_t>, grid, dim3(256), 0, stream, gu, nsplit, split_stride, bias,
                       (bf16_t*)out, count, f, act, limit, alpha);
  else
    hipLaunchKernelGGL(gate_bias_kernel<float>, grid, dim3(256), 0, stream, gu, nsplit, split_stride, bias, (float*)out,
                       count, f, act, limit, alpha);
  KLLM_CHECK_LAUNCH("gate_bias");
  return 0;
}
