// Causal attention over the paged cache, one workgroup per (token, head):
// the kernel that takes every size and both dtypes.  The faster kernels for
// prompts and for decode batches are tested against it.
//
// For the token at position p of its request, head h reads KV head
// h / (H/KV) and the keys [max(0, p - window + 1), p] (all keys [0, p] when
// window is 0): reference backend/model.cu:343-408 (scores, maximum, exp,
// sum, values) and :224-225 (window).  Unlike the reference, which keeps all
// scores of a row in shared memory, scores are taken 256 keys at a time with
// a running maximum and sum, so the context is not bounded by a buffer.
//
// Options that a design may ask for: values of another width than the keys
// (vd); a chunked mask (chunk > 0: the query at p reads no key before
// p - p % chunk, chunks counted from position 0 of the request); a sink
// (sink != 0: the softmax's denominator has one more term, exp(0), a key whose
// score is 0 and whose value is nothing); kept first positions (keep_first > 0: the first
// keep_first positions of a request stay readable behind the window, at their true places).
//
// Page layout: keys [KV][slot][hd], then values [KV][vd][slot].
#include <math.h>

#include "common.hpp"
#include "kllm_kernels.h"

namespace kllm {

constexpr int kAttnThreads = 256;
constexpr int kMaxHeadDim = 256;

template <typename T>
__global__ __launch_bounds__(kAttnThreads) void attn_generic_kernel(
    const T* __restrict__ q, T* __restrict__ out, const T* __restrict__ cache,
    const int* __restrict__ positions, const int* __restrict__ span_of_token,
    const int* __restrict__ block_table, int max_pages, int page_size, int H, int KV, int hd,
    int vd, int window, int chunk, int sink, float scale, const float* __restrict__ slopes, int keep_first) {
  __shared__ float qs[kMaxHeadDim];
  __shared__ float ps[kAttnThreads];
  __shared__ float red[16];
  __shared__ float part[kAttnThreads];

  const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int kvh = h / (H / KV);
  const int pos = positions[t];
  const int len = pos + 1;
  const float slope = slopes ? slopes[h] : 0.f;   // a bias that grows with the distance to the key
  const int start = first_key(pos, window, chunk);
  const int* table = block_table + (long)span_of_token[t] * max_pages;
  const long kblock = (long)page_size * hd, vblock = (long)page_size * vd;
  const long page_elems = (long)KV * (kblock + vblock);

  const T* qrow = q + ((long)t * H + h) * hd;
  for (int i = tid; i < hd; i += kAttnThreads) qs[i] = to_f32(qrow[i]);
  __syncthreads();

  // Values: thread (d, sl) sums over the pages sl, sl + nslice, ... of a chunk.
  const int nslice = kAttnThreads / vd;
  const int d = tid % vd, sl = tid / vd;
  const bool pv_thread = sl < nslice;

  const int chunk_pages = page_size >= kAttnThreads ? 1 : kAttnThreads / page_size;
  const int chunk_keys = chunk_pages * page_size;  // <= 256 (page_size <= 256 is checked on the host)

  float m = -INFINITY, l = 0.f, acc = 0.f;
  // Two runs of keys: the kept first positions that lie behind the window (none without
  // keep_first), then the window itself.  Pages between the two may have been given back.
  const int kept = min(keep_first, start);
  for (int run = kept > 0 ? 0 : 1; run < 2; ++run) {
  const int lo_key = run == 0 ? 0 : start, hi_key = run == 0 ? kept : len;
  for (int pg0 = lo_key / page_size; pg0 * page_size < hi_key; pg0 += chunk_pages) {
    const int base = pg0 * page_size;
    // ---- scores of this chunk: thread i <-> key base + i
    float s = -INFINITY;
    const int key = base + tid;
    if (tid < chunk_keys && key >= lo_key && key < hi_key) {
      const int page = table[key / page_size];
      const T* krow = cache + page * page_elems + kvh * kblock + (long)(key % page_size) * hd;
      float dot = 0.f;
      for (int i = 0; i < hd; ++i) dot = fmaf(qs[i], to_f32(krow[i]), dot);
      s = dot * scale - slope * (float)(pos - key);
    }
    const float cmax = block_max(s, red);
    const float m_new = fmaxf(m, cmax);
    const float alpha = expf(m - m_new);  // 0 on the first chunk (m = -inf)
    const float p = (s == -INFINITY) ? 0.f : expf(s - m_new);
    ps[tid] = p;
    const float csum = block_sum(p, red);  // its barriers also publish ps
    l = l * alpha + csum;
    m = m_new;
    acc *= alpha;
    // ---- values
    if (pv_thread) {
      for (int pg = sl; pg < chunk_pages; pg += nslice) {
        const int pbase = base + pg * page_size;
        const int lo = max(lo_key - pbase, 0), hi = min(hi_key - pbase, page_size);
        if (lo >= hi) continue;
        const int page = table[pbase / page_size];
        const T* vrow = cache + page * page_elems + KV * kblock + kvh * vblock + (long)d * page_size;
        const float* pp = ps + pg * page_size;
        for (int sidx = lo; sidx < hi; ++sidx) acc = fmaf(pp[sidx], to_f32(vrow[sidx]), acc);
      }
    }
    __syncthreads();  // ps is rewritten by the next chunk
  }
  }

  if (sink) {   // one more key whose score is 0: it joins the sum, and nothing else
    const float m_all = fmaxf(m, 0.f);
    const float alpha = expf(m - m_all);
    l = l * alpha + expf(-m_all);
    acc *= alpha;
  }
  part[tid] = pv_thread ? acc : 0.f;
  __syncthreads();
  if (tid < vd) {
    float o = 0.f;
    for (int s2 = 0; s2 < nslice; ++s2) o += part[s2 * vd + tid];
    out[((long)t * H + h) * vd + tid] = from_f32<T>(o / l);
  }
}

}  // namespace kllm

using namespace kllm;

extern "C" int kllm_attn_generic(const void* q, void* out, const void* cache, const int* positions,
                                 const int* span_of_token, const int* block_table, int max_pages,
                                 int page_size, int n, int H, int KV, int hd, int vd, int window,
                                 int chunk, int sink, float scale, const float* slopes, int dtype,
                                 int keep_first, hipStream_t stream) {
  KLLM_REQUIRE(q && out && cache && positions && span_of_token && block_table,
               "attn_generic: null pointer");
  KLLM_REQUIRE(n > 0 && H > 0 && KV > 0 && H % KV == 0, "attn_generic: bad heads n=%d H=%d KV=%d", n,
               H, KV);
  KLLM_REQUIRE(hd > 0 && hd <= kMaxHeadDim, "attn_generic: head_dim %d is outside [1, %d]", hd,
               kMaxHeadDim);
  KLLM_REQUIRE(page_size > 0 && page_size <= kAttnThreads && max_pages > 0,
               "attn_generic: page_size %d is outside [1, %d]", page_size, kAttnThreads);
  KLLM_REQUIRE(vd > 0 && vd <= kMaxHeadDim, "attn_generic: value width %d is outside [1, %d]", vd, kMaxHeadDim);
  KLLM_REQUIRE(window >= 0 && chunk >= 0 && keep_first >= 0, "attn_generic: negative window, chunk or keep_first");
  KLLM_REQUIRE(H <= 65535, "attn_generic: too many heads for the grid");
  KLLM_REQUIRE(dtype == DT_F32 || dtype == DT_BF16, "attn_generic: unknown dtype %d", dtype);
  const dim3 grid(n, H);
  if (dtype == DT_F32)
    hipLaunchKernelGGL(attn_generic_kernel<float>, grid, dim3(kAttnThreads), 0, stream,
                       (const float*)q, (float*)out, (const float*)cache, positions, span_of_token,
                       block_table, max_pages, page_size, H, KV, hd, vd, window, chunk, sink, scale, slopes, keep_first);
  else
    hipLaunchKernelGGL(attn_generic_kernel<bf16_t>, grid, dim3(kAttnThreads), 0, stream,
                       (const bf16_t*)q, (bf16_t*)out, (const bf16_t*)cache, positions,
                       span_of_token, block_table, max_pages, page_size, H, KV, hd, vd, window, chunk, sink, scale, slopes, keep_first);
  KLLM_CHECK_LAUNCH("attn_generic");
  return 0;
}
