// A recurrent mixer with a matrix state per head, updated by a generalized delta rule:
//
//   S_t = diag(w_t) S_(t-1) - (a_t * u_t) (u_t^T S_(t-1)) + k_t v_t^T        o_t = S_t^T r_t
//
// with u_t the key divided by its length, w_t a decay per key channel and a_t a removal rate
// per key channel.  S is [key channel][value channel], 32-bit, one per request and head, kept
// in a state slot between steps and started from zero at position 0.
//
// Three kernels: `prep` turns the projections' sums into what the recurrence reads (per token,
// parallel), `scan` runs the recurrence (per request and head, token after token), `out`
// normalises each head's output, scales and gates it (per token, parallel).  Everything that
// enters the recurrence is 32-bit.
#include <math.h>

#include "common.hpp"
#include "kllm_kernels.h"

namespace kllm {

constexpr int kPrepThreads = 256;
// per (token, head): r, k, v, w, u, a*u, each hd floats
constexpr int kScanFields = 6;

// proj: [nsplit][n][5*HD + L], columns r | k | v | g | a | w1.
// scan_in: [H][n][6][hd] (a head's tokens follow each other, as the scan reads them); gate: [n][HD] = sigmoid(g).
// A workgroup takes one token and as many whole heads as its threads hold channels
// (blockIdx.y), a thread one channel: every load of a thread is independent of the others.
template <typename TW>
__global__ __launch_bounds__(kPrepThreads) void delta_prep_kernel(
    const float* __restrict__ proj, int nsplit, long split_stride, const float* __restrict__ a_bias,
    const TW* __restrict__ w2, const float* __restrict__ w0, const float* __restrict__ low, int low_nsplit,
    long low_stride, float decay_scale, float key_eps, float* __restrict__ scan_in, float* __restrict__ gate, int H,
    int hd, int L, int heads_per_wg) {
  extern __shared__ float lds[];           // [L] tanh of the low-rank input, [heads_per_wg * hd] squares of the keys
  float* tl = lds;
  float* ksq = lds + L;
  const int t = blockIdx.x, tid = threadIdx.x;
  const int HD = H * hd, cols = 5 * HD + L;
  const float* in = proj + (long)t * cols;
  const int h = blockIdx.y * heads_per_wg + tid / hd, e = tid % hd;
  const bool live = tid < heads_per_wg * hd && h < H;
  const int c = live ? h * hd + e : 0;
  if (!low)
    for (int l = tid; l < L; l += kPrepThreads) {
      float v = 0.f;
      for (int s = 0; s < nsplit; ++s) v += in[5 * HD + l + s * split_stride];
      tl[l] = tanhf(v);
    }
  float f[5] = {0.f, 0.f, 0.f, 0.f, 0.f};  // r, k, v, g, a
  for (int s = 0; s < nsplit; ++s)
#pragma unroll
    for (int q = 0; q < 5; ++q) f[q] += in[q * HD + c + s * split_stride];
  float lr = w0[c];
  const float ab = a_bias[c];
  if (low)
    for (int sl = 0; sl < low_nsplit; ++sl) lr += low[(long)t * HD + c + sl * low_stride];
  ksq[tid] = live ? f[1] * f[1] : 0.f;
  __syncthreads();
  if (!low) {
    if (L % 8 == 0 && (((uintptr_t)w2) & 15) == 0) {          // the row in 16- or 32-byte loads, all in flight
      typedef TW row8 __attribute__((ext_vector_type(8)));
      const row8* w2r = reinterpret_cast<const row8*>(w2 + (long)c * L);
      float l0 = 0.f, l1 = 0.f;
#pragma unroll 4
      for (int l8 = 0; l8 < L / 8; ++l8) {
        const row8 wv = w2r[l8];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          l0 = fmaf(to_f32(wv[q]), tl[8 * l8 + q], l0);
          l1 = fmaf(to_f32(wv[4 + q]), tl[8 * l8 + 4 + q], l1);
        }
      }
      lr += l0 + l1;
    } else {
      const TW* w2r = w2 + (long)c * L;
      for (int l = 0; l < L; ++l) lr = fmaf(to_f32(w2r[l]), tl[l], lr);
    }
  }
  float kss = 0.f;                         // the head's sum of squares, in the order of its channels
  const float* hsq = ksq + (tid / hd) * hd;
  for (int q = 0; q < hd; ++q) kss += hsq[q];
  if (!live) return;
  const float w = expf(-decay_scale * sigmoid_f32(lr));
  const float a = sigmoid_f32(f[4] + ab);
  const float u = f[1] / sqrtf(kss + key_eps);
  float* o = scan_in + (((long)h * gridDim.x + t) * kScanFields) * hd + e;
  o[0 * hd] = f[0];
  o[1 * hd] = f[1];
  o[2 * hd] = f[2];
  o[3 * hd] = w;
  o[4 * hd] = u;
  o[5 * hd] = a * u;
  gate[(long)t * HD + c] = sigmoid_f32(f[3]);
}

constexpr int kScanThreads = 256;
constexpr int kScanWaves = kScanThreads / kWave;

// The recurrence.  Columns of the state (value channels) do not see each other, so a workgroup
// takes a block of columns of one (span, head): thread (j, p) holds rows [NR p, NR p + NR) of
// column j, the PARTS threads of a column are neighbouring lanes of one wave.  A token's vectors
// are the same for every column; they are staged through LDS a block of tokens at a time (32
// tokens for heads up to 64): the next block's loads from memory are all asked for before this
// block's tokens are worked through and put into LDS behind them, so the memory's latency hides
// behind a block's arithmetic (it did not behind 8 tokens'), and the chain from token to token
// holds arithmetic and LDS reads only.  A block's code has no branch: a span that ends inside
// a block is filled with tokens that change nothing (decay one, everything else zero).  Rows
// beyond hd are padding: their vectors are zero in LDS and their state stays zero.
template <int PARTS, int NR>
__global__ __launch_bounds__(kScanThreads) void delta_scan_kernel(
    const float* __restrict__ scan_in, float* __restrict__ o_out, float* __restrict__ state,
    const int* __restrict__ slots, const int* __restrict__ span_start, const int* __restrict__ span_pos, int n,
    int H, int hd) {
  static_assert(NR % 4 == 0, "rows in fours");
  constexpr int HP = PARTS * NR;                       // rows with padding
  constexpr int COLS = kScanThreads / PARTS;           // columns of a workgroup
  constexpr int TB = 2048 / HP < 32 ? 2048 / HP : 32;  // tokens of a block
  constexpr int KEEPS = (TB + PARTS - 1) / PARTS;      // outputs a lane keeps: token tt's lies in lane tt % PARTS
  constexpr int VEC = kScanFields * HP;                // floats of a token in LDS
  constexpr int EPL = (VEC + kWave - 1) / kWave;       // elements of a token that a lane stages
  constexpr int TPW = TB / kScanWaves;                 // tokens of a block that a wave stages
  static_assert(TB % kScanWaves == 0 && TB * VEC * sizeof(float) <= 48 * 1024, "a block is staged by whole waves");
  __shared__ __attribute__((aligned(16))) float tok[TB * VEC];
  const int span = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int lane = tid % kWave, wave = tid / kWave;
  const int j = blockIdx.z * COLS + tid / PARTS, p = tid % PARTS;
  const bool col = j < hd;
  const int row0 = p * NR;
  float* S = state + ((long)slots[span] * H + h) * hd * hd;
  const int t0 = span_start[span], t1 = span_start[span + 1];
  const bool fresh = span_pos[span] == 0;
  float s[NR];
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int r = row0 + i;
    s[i] = (col && r < hd && !fresh) ? S[(long)r * hd + j] : 0.f;
  }
  if (HP != hd)
    for (int i = tid; i < TB * VEC; i += kScanThreads) tok[i] = 0.f;
  // Staging: wave w takes the block's tokens w, w + 4, ...; a lane the elements lane, lane + 64,
  // ... of a token.  Where an element goes in LDS, and what stands there for a token that does
  // not exist, is worked out once.
  const int per_tok = kScanFields * hd;                // floats of a token in memory
  const long tok_stride = per_tok;                     // a head's tokens follow each other
  const float* base = scan_in + (long)h * n * per_tok;
  int from_e[EPL], to_e[EPL];
  float pad_e[EPL];
#pragma unroll
  for (int i = 0; i < EPL; ++i) {
    const int e = lane + i * kWave;
    from_e[i] = e < per_tok ? e : 0;                   // (an element beyond the token reads a place that exists)
    to_e[i] = e < per_tok ? (e / hd) * HP + e % hd : -1;
    pad_e[i] = e / hd == 3 ? 1.f : 0.f;
  }
  float pre[TPW * EPL];
  // Every load is made, none inside a branch: an element of a token that does not exist reads a
  // token that does, and is dropped when the block is put into LDS.
  auto ask = [&](int first) {
#pragma unroll
    for (int q = 0; q < TPW; ++q) {
      const int t = min(first + wave + q * kScanWaves, t1 - 1);
      const float* src = base + (long)t * tok_stride;
#pragma unroll
      for (int i = 0; i < EPL; ++i) pre[q * EPL + i] = src[from_e[i]];
    }
  };
  auto put = [&](int first) {
#pragma unroll
    for (int q = 0; q < TPW; ++q) {
      const int tt = wave + q * kScanWaves;
      const bool there = first + tt < t1;
#pragma unroll
      for (int i = 0; i < EPL; ++i)
        if (to_e[i] >= 0) tok[tt * VEC + to_e[i]] = there ? pre[q * EPL + i] : pad_e[i];
    }
  };
  auto lds_barrier = [&]() {   // orders LDS traffic only: loads from memory stay in flight
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0xC07F);
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };
  __syncthreads();                                     // the padding is zero before anything is staged
  ask(t0);
  put(t0);
  __syncthreads();
  const long o_step = (long)H * hd;
  float o_keep[KEEPS];
  struct TokenVectors {                                // this thread's rows of a token's vectors
    floatx4 u[NR / 4], w[NR / 4], k[NR / 4], a[NR / 4], r[NR / 4];
    float vj;
  };
  auto fetch = [&](const float* tv) {
    TokenVectors T;
#pragma unroll
    for (int c = 0; c < NR / 4; ++c) {
      T.u[c] = *reinterpret_cast<const floatx4*>(tv + 4 * HP + row0 + 4 * c);
      T.w[c] = *reinterpret_cast<const floatx4*>(tv + 3 * HP + row0 + 4 * c);
      T.k[c] = *reinterpret_cast<const floatx4*>(tv + HP + row0 + 4 * c);
      T.a[c] = *reinterpret_cast<const floatx4*>(tv + 5 * HP + row0 + 4 * c);
      T.r[c] = *reinterpret_cast<const floatx4*>(tv + row0 + 4 * c);
    }
    T.vj = tv[2 * HP + (col ? j : 0)];
    return T;
  };
  auto token = [&](int tt, const TokenVectors& T) {
    float us0 = 0.f, us1 = 0.f;
#pragma unroll
    for (int c = 0; c < NR / 4; ++c) {
      us0 = fmaf(T.u[c][0], s[4 * c], us0);
      us1 = fmaf(T.u[c][1], s[4 * c + 1], us1);
      us0 = fmaf(T.u[c][2], s[4 * c + 2], us0);
      us1 = fmaf(T.u[c][3], s[4 * c + 3], us1);
    }
    const float us = parts_sum<PARTS>(us0 + us1);
    float o0 = 0.f, o1 = 0.f;
#pragma unroll
    for (int c = 0; c < NR / 4; ++c)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float sn = fmaf(T.w[c][e], s[4 * c + e], fmaf(T.k[c][e], T.vj, -T.a[c][e] * us));
        s[4 * c + e] = sn;
        if (e % 2 == 0) o0 = fmaf(sn, T.r[c][e], o0); else o1 = fmaf(sn, T.r[c][e], o1);
      }
    const float o_sum = parts_sum<PARTS>(o0 + o1);     // not part of the chain from token to token
    o_keep[tt / PARTS] = p == tt % PARTS ? o_sum : o_keep[tt / PARTS];
  };
  for (int tb = t0; tb < t1; tb += TB) {
    ask(tb + TB);                                      // the next block, on its way during this one
    TokenVectors cur = fetch(tok);
#pragma unroll
    for (int tt = 0; tt < TB; ++tt) {
      const TokenVectors nxt = fetch(tok + (tt + 1 < TB ? tt + 1 : tt) * VEC);
      token(tt, cur);
      cur = nxt;
    }
#pragma unroll
    for (int q = 0; q < KEEPS; ++q) {
      const int t = tb + q * PARTS + p;
      if (col && q * PARTS + p < TB && t < t1) o_out[(long)t * o_step + h * hd + j] = o_keep[q];
    }
    lds_barrier();                                     // everybody is done with this block
    put(tb + TB);
    lds_barrier();                                     // the next block is staged
  }
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int r = row0 + i;
    if (col && r < hd) S[(long)r * hd + j] = s[i];
  }
}

// out[t][h*hd + e] = o / sqrt(mean over the head of o^2 + eps) * weight * gate, one wave per (token, head).
template <typename T>
__global__ void delta_out_kernel(const float* __restrict__ o, const float* __restrict__ gate,
                                 const float* __restrict__ weight, float eps, T* __restrict__ out, long heads_total,
                                 int H, int hd) {
  const long item = (long)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (item >= heads_total) return;
  const int lane = threadIdx.x % kWave;
  const int h = (int)(item % H);
  const float* orow = o + item * hd;
  float ss = 0.f;
  for (int e = lane; e < hd; e += kWave) ss = fmaf(orow[e], orow[e], ss);
  ss = wave_sum(ss);
  const float rstd = 1.f / sqrtf(ss / (float)hd + eps);
  for (int e = lane; e < hd; e += kWave)
    out[item * hd + e] = from_f32<T>(orow[e] * rstd * weight[h * hd + e] * gate[item * hd + e]);
}

}  // namespace kllm

using namespace kllm;

extern "C" int kllm_delta_prep(const float* proj, int nsplit, long split_stride, const float* a_bias, const void* w2,
                               const float* w0, const float* low, int low_nsplit, long low_stride, float decay_scale,
                               float key_eps, float* scan_in, float* gate, int n, int H, int hd, int L, int w_dtype,
                               hipStream_t stream) {
  KLLM_REQUIRE(proj && a_bias && (w2 || low) && w0 && scan_in && gate, "delta_prep: null pointer");
  KLLM_REQUIRE(!low || low_nsplit >= 1, "delta_prep: the low-rank sums need at least one slice");
  KLLM_REQUIRE(n > 0 && H > 0 && hd > 0 && L > 0 && nsplit >= 1, "delta_prep: bad sizes n=%d H=%d hd=%d L=%d", n, H, hd,
               L);
  KLLM_REQUIRE(w_dtype == DT_F32 || w_dtype == DT_BF16, "delta_prep: unknown dtype %d", w_dtype);
  KLLM_REQUIRE(hd <= kPrepThreads, "delta_prep: heads of %d are not built (up to %d)", hd, kPrepThreads);
  const int heads_per_wg = kPrepThreads / hd < H ? kPrepThreads / hd : H;
  const size_t lds = ((size_t)L + kPrepThreads) * sizeof(float);
  KLLM_REQUIRE(lds <= 64 * 1024, "delta_prep: a low-rank width of %d does not fit into LDS", L);
  const dim3 grid(n, ceil_div(H, heads_per_wg));
  KLLM_REQUIRE(grid.y <= 65535, "delta_prep: too many heads for the grid");
  if (w_dtype == DT_F32)
    hipLaunchKernelGGL(delta_prep_kernel<float>, grid, dim3(kPrepThreads), lds, stream, proj, nsplit, split_stride,
                       a_bias, (const float*)w2, w0, low, low_nsplit, low_stride, decay_scale, key_eps, scan_in, gate,
                       H, hd, L, heads_per_wg);
  else
    hipLaunchKernelGGL(delta_prep_kernel<bf16_t>, grid, dim3(kPrepThreads), lds, stream, proj, nsplit, split_stride,
                       a_bias, (const bf16_t*)w2, w0, low, low_nsplit, low_stride, decay_scale, key_eps, scan_in, gate,
                       H, hd, L, heads_per_wg);
  KLLM_CHECK_LAUNCH("delta_prep");
  return 0;
}

extern "C" int kllm_delta_scan_max_dim(void) { return 256; }

extern "C" int kllm_delta_scan(const float* scan_in, float* o_out, float* state, const int* slots,
                               const int* span_start, const int* span_pos, int n_spans, int n, int H, int hd,
                               hipStream_t stream) {
  KLLM_REQUIRE(n > 0, "delta_scan: no tokens");
  KLLM_REQUIRE(scan_in && o_out && state && slots && span_start && span_pos, "delta_scan: null pointer");
  KLLM_REQUIRE(n_spans > 0 && H > 0 && H <= 65535 && hd > 0 && hd <= 256, "delta_scan: bad sizes spans=%d H=%d hd=%d",
               n_spans, H, hd);
  // A column's rows over neighbouring lanes, four to a lane for heads up to 64 and eight above
  // (sixteen lanes sum by data-parallel moves alone; more need a lane exchange through LDS on
  // the chain from token to token): 4, 8 ... 64 rows with padding, then 128, 256.
  const int nr = hd > 64 ? 8 : 4;
  int parts = 1;
  while (parts * nr < hd) parts *= 2;
  const int cols = kScanThreads / parts;
  const dim3 grid(n_spans, H, ceil_div(hd, cols));
#define KLLM_SCAN(PARTS, NR)                                                                                       \
  hipLaunchKernelGGL((delta_scan_kernel<PARTS, NR>), grid, dim3(kScanThreads), 0, stream, scan_in, o_out, state, \
                     slots, span_start, span_pos, n, H, hd)
  if (nr == 4) {
    switch (parts) {
      case 1: KLLM_SCAN(1, 4); break;
      case 2: KLLM_SCAN(2, 4); break;
      case 4: KLLM_SCAN(4, 4); break;
      case 8: KLLM_SCAN(8, 4); break;
      default: KLLM_SCAN(16, 4); break;
    }
  } else {
    if (parts <= 16) KLLM_SCAN(16, 8); else KLLM_SCAN(32, 8);
  }
#undef KLLM_SCAN
  KLLM_CHECK_LAUNCH("delta_scan");
  return 0;
}

extern "C" int kllm_delta_out(const float* o, const float* gate, const float* weight, float eps, void* out, int n, int H,
                              int hd, int dtype, hipStream_t stream) {
  KLLM_REQUIRE(o && gate && weight && out, "delta_out: null pointer");
  KLLM_REQUIRE(n > 0 && H > 0 && hd > 0, "delta_out: bad sizes n=%d H=%d hd=%d", n, H, hd);
  KLLM_REQUIRE(dtype == DT_F32 || dtype == DT_BF16, "delta_out: unknown dtype %d", dtype);
  const long total = (long)n * H;
  const dim3 grid(ceil_div(total, 4));
  if (dtype == DT_F32)
    hipLaunchKernelGGL(delta_out_kernel<float>, grid, dim3(256), 0, stream, o, gate, weight, eps, (float*)out, total, H,
                       hd);
  else
    hipLaunchKernelGGL(delta_out_kernel<bf16_t>, grid, dim3(256), 0, stream, o, gate, weight, eps, (bf16_t*)out, total,
                       H, hd);
  KLLM_CHECK_LAUNCH("delta_out");
  return 0;
}
