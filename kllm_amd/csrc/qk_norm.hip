// What lies between the query/key product and attention for a mixer whose queries and keys
// are normalised over the whole projection: biases, an RMS norm over the whole query
// projection and one over the whole key projection (all heads at once), a rotation of the
// first `rot` elements of every head behind the norm, a query temperature that grows with
// the position, and the append to the pages.  Without values of its own (dv == 0) the key as
// projected (bias added, before its norm) is cached as the value, its normalised form as the
// key; with them (dv > 0) the sums hold KV * dv value columns behind the keys.  One workgroup
// per token, all in 32-bit.
//
// Page layout: keys [KV][slot][hd], then values [KV][dv][slot] (dv == 0: values as wide as keys).
#include <math.h>

#include "common.hpp"
#include "kllm_kernels.h"

namespace kllm {

constexpr int kQkThreads = 256;

template <typename T>
__global__ __launch_bounds__(kQkThreads) void qk_norm_append_kernel(
    const float* __restrict__ qk, int nsplit, long split_stride, const float* __restrict__ q_bias,
    const float* __restrict__ k_bias, const float* __restrict__ q_w, const float* __restrict__ k_w, float eps,
    float temp_coef, int temp_every, T* __restrict__ q_out, T* __restrict__ cache, const int* __restrict__ positions,
    const int* __restrict__ span_of_token, const int* __restrict__ block_table, int max_pages, int page_size, int H,
    int KV, int hd, int dv, const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rot, int interleaved) {
  extern __shared__ float row[];            // [H*hd + KV*hd + KV*dv] the sums, then as many norm weights
  __shared__ float red[16];
  const int t = blockIdx.x, tid = threadIdx.x;
  const int qd = H * hd, kd = KV * hd, cols = qd + kd + KV * dv;
  const float* in = qk + (long)t * cols;
  float* wrow = row + cols;
  float ssq = 0.f, ssk = 0.f;
  // eight of a thread's elements at a time: their loads (every slice, the bias) go out together
  for (int i0 = tid; i0 < cols; i0 += 8 * kQkThreads) {
    float v[8], wv[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = i0 + u * kQkThreads;
      v[u] = 0.f;
      wv[u] = 1.f;
      if (i < cols) {
        if (i < qd) {
          if (q_w) wv[u] = q_w[i];
        } else if (k_w && i < qd + kd) {
          wv[u] = k_w[i - qd];
        }
        if (i < qd) {
          if (q_bias) v[u] = q_bias[i];
        } else if (k_bias && i < qd + kd) {
          v[u] = k_bias[i - qd];
        }
      }
    }
    for (int s = 0; s < nsplit; ++s)
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int i = i0 + u * kQkThreads;
        v[u] += i < cols ? in[i + s * split_stride] : 0.f;
      }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = i0 + u * kQkThreads;
      if (i >= cols) continue;
      if (i < qd) ssq = fmaf(v[u], v[u], ssq); else if (i < qd + kd) ssk = fmaf(v[u], v[u], ssk);
      row[i] = v[u];
      wrow[i] = wv[u];
    }
  }
  ssq = block_sum(ssq, red);
  ssk = block_sum(ssk, red);
  const int pos = positions[t];
  float qmul = 1.f;
  if (temp_every > 0) qmul = 1.f + temp_coef * logf((float)((pos + 1) / temp_every) + 1.f);
  const float rq = q_w ? 1.f / sqrtf(ssq / (float)qd + eps) : 1.f;
  const float rk = k_w ? 1.f / sqrtf(ssk / (float)kd + eps) : 1.f;
  // Element i of the normalised query (base 0) or key (base qd) projection, turned with its
  // partner where it lies among the first `rot` elements of its head.
  const int rhalf = rot / 2;
  auto normed = [&](int base, int i, float rs, bool weighted) {
    const float v = row[base + i];
    return weighted ? v * rs * wrow[base + i] : v;
  };
  auto turned = [&](int base, int i, float rs, bool weighted) {
    const float v = normed(base, i, rs, weighted);
    const int e = i % hd;
    if (!cos_t || e >= rot) return v;
    int j, partner;
    bool first;
    if (interleaved) {
      j = e / 2;
      first = (e & 1) == 0;
      partner = first ? i + 1 : i - 1;
    } else {
      first = e < rhalf;
      j = first ? e : e - rhalf;
      partner = first ? i + rhalf : i - rhalf;
    }
    const float o = normed(base, partner, rs, weighted);
    const float c = cos_t[(long)t * rhalf + j], sn = sin_t[(long)t * rhalf + j];
    return first ? v * c - o * sn : v * c + o * sn;
  };
#pragma unroll 4
  for (int i = tid; i < qd; i += kQkThreads)
    q_out[(long)t * qd + i] = from_f32<T>(turned(0, i, rq, q_w != nullptr) * qmul);
  if (!cache) return;
  const int page = block_table[(long)span_of_token[t] * max_pages + pos / page_size];
  const int slot = pos % page_size;
  const int vw = dv > 0 ? dv : hd;           // a value's width
  const long kblock = (long)page_size * hd, vblock = (long)page_size * vw;
  T* page_base = cache + (long)page * KV * (kblock + vblock);
  for (int i = tid; i < kd; i += kQkThreads) {
    const int kvh = i / hd, e = i % hd;
    page_base[kvh * kblock + (long)slot * hd + e] = from_f32<T>(turned(qd, i, rk, k_w != nullptr));
    if (dv == 0) page_base[KV * kblock + kvh * vblock + (long)e * page_size + slot] = from_f32<T>(row[qd + i]);
  }
  for (int i = tid; i < KV * dv; i += kQkThreads) {
    const int kvh = i / dv, e = i % dv;
    page_base[KV * kblock + kvh * vblock + (long)e * page_size + slot] = from_f32<T>(row[qd + kd + i]);
  }
}

}  // namespace kllm

using namespace kllm;

extern "C" int kllm_qk_norm_append(const float* qk, int nsplit, long split_stride, const float* q_bias,
                                   const float* k_bias, const float* q_w, const float* k_w, float eps, float temp_coef,
                                   int temp_every, void* q_out, void* cache, const int* positions,
                                   const int* span_of_token, const int* block_table, int max_pages, int page_size,
                                   int n, int H, int KV, int hd, int dtype, int dv, const float* cos_t,
                                   const float* sin_t, int rot, int interleaved, hipStream_t stream) {
  KLLM_REQUIRE(qk && q_out && positions, "qk_norm_append: null pointer");
  KLLM_REQUIRE(!cache || (span_of_token && block_table && max_pages > 0 && page_size > 0),
               "qk_norm_append: a cache needs its tables");
  KLLM_REQUIRE(n > 0 && H > 0 && KV > 0 && hd > 0 && nsplit >= 1, "qk_norm_append: bad sizes n=%d H=%d KV=%d hd=%d", n,
               H, KV, hd);
  KLLM_REQUIRE(dtype == DT_F32 || dtype == DT_BF16, "qk_norm_append: unknown dtype %d", dtype);
  KLLM_REQUIRE(dv >= 0 && (cos_t == nullptr) == (sin_t == nullptr), "qk_norm_append: dv %d, or cos without sin", dv);
  KLLM_REQUIRE(!cos_t || (rot > 0 && rot % 2 == 0 && rot <= hd && (interleaved == 0 || interleaved == 1)),
               "qk_norm_append: rotary dimension %d of a head of %d", rot, hd);
  const size_t lds = 2 * ((size_t)(H + KV) * hd + (size_t)KV * dv) * sizeof(float);
  KLLM_REQUIRE(lds <= 160 * 1024, "qk_norm_append: %d query and key channels do not fit into LDS", (H + KV) * hd);
  if (lds > 64 * 1024) {
    const void* fn = dtype == DT_F32 ? (const void*)qk_norm_append_kernel<float> : (const void*)qk_norm_append_kernel<bf16_t>;
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) KLLM_FAIL((int)e, "qk_norm_append: cannot raise the LDS limit: %s", hipGetErrorString(e));
  }
  if (dtype == DT_F32)
    hipLaunchKernelGGL(qk_norm_append_kernel<float>, dim3(n), dim3(kQkThreads), lds, stream, qk, nsplit, split_stride,
                       q_bias, k_bias, q_w, k_w, eps, temp_coef, temp_every, (float*)q_out, (float*)cache, positions,
                       span_of_token, block_table, max_pages, page_size, H, KV, hd, dv, cos_t, sin_t, rot, interleaved);
  else
    hipLaunchKernelGGL(qk_norm_append_kernel<bf16_t>, dim3(n), dim3(kQkThreads), lds, stream, qk, nsplit, split_stride,
                       q_bias, k_bias, q_w, k_w, eps, temp_coef, temp_every, (bf16_t*)q_out, (bf16_t*)cache, positions,
                       span_of_token, block_table, max_pages, page_size, H, KV, hd, dv, cos_t, sin_t, rot, interleaved);
  KLLM_CHECK_LAUNCH("qk_norm_append");
  return 0;
}
