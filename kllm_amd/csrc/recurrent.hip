// Recurrent mixers whose state is carried from token to token, and what they share.
//
// A short causal convolution per channel: y_t = sum_j w[c][j] x_(t - taps + 1 + j), zeros before
// position 0.  Its inputs of the last taps - 1 positions are part of a request's state: the
// kernels that convolve read them for the first tokens of a span, and `conv_state_update`, a
// launch of its own behind them, writes the span's last inputs there (one thread per request
// and channel reads the old entries before it writes the new ones).
//
// The gated delta rule, per head with a state S [key channel][value channel]:
//
//   S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
//
// with q and k unit vectors per head (q also times dk^-1/2), g = exp(-exp(A) softplus(a + dt))
// and beta = sigmoid(b).  `gated_delta_prep` turns the projections' sums into these (per token,
// parallel: convolution and SiLU of q, k, v, the unit norms, g, beta and the output gate),
// `gated_delta_scan` runs the recurrence (per request, head and block of value channels, token
// after token); the output's norm and gate are kllm_delta_out's.
//
// The gated linear recurrence, per channel: with u the convolved input, gates
// r = sigmoid(A_r u + b_r), i = sigmoid(A_i u + b_i) through block-diagonal matrices,
// log a = -c r (c = 8 softplus(lambda), prepared once), S <- a S + sqrt(1 - a^2) i u, and the
// output S * gelu(y) with y a second branch.  `linear_recurrence_prep` makes a and the added term
// for every token (parallel), `linear_recurrence_scan` runs the chain.
//
// States are 32-bit and start from zero where a span's first position is 0.  Everything here
// computes in 32-bit from the projections' 32-bit sums.
#include <math.h>

#include "common.hpp"
#include "kllm_kernels.h"

namespace kllm {

constexpr int kRecThreads = 256;
constexpr int kMaxTaps = 16;

// The input of the convolution at row `row` of the step (a token of the same span), channel c.
__device__ __forceinline__ float conv_input(const float* __restrict__ proj, int nsplit, long split_stride, long cols,
                                            long col, const float* __restrict__ bias, long row) {
  const float* p = proj + row * cols + col;
  float v = 0.f;
  for (int s = 0; s < nsplit; ++s) v += p[s * split_stride];
  return bias ? v + bias[col] : v;
}

// The convolution's output for the token at row t (span rows from t0, `fresh`: the span starts at
// position 0), channel c of C, whose input column is col0 + c; `st` is the request's
// [C][taps - 1] entries.
__device__ __forceinline__ float conv_at(const float* __restrict__ proj, int nsplit, long split_stride, long cols,
                                         long col, const float* __restrict__ in_bias,
                                         const float* __restrict__ w_row, int taps, const float* __restrict__ st_row,
                                         bool fresh, long t, long t0) {
  float y = 0.f;
  const int K = taps - 1;
  for (int j = 0; j < taps; ++j) {
    const long row = t - K + j;
    float x;
    if (row >= t0) x = conv_input(proj, nsplit, split_stride, cols, col, in_bias, row);
    else x = fresh ? 0.f : st_row[K - (int)(t0 - row)];
    y = fmaf(w_row[j], x, y);
  }
  return y;
}

__global__ __launch_bounds__(kRecThreads) void conv_state_update_kernel(
    const float* __restrict__ proj, int nsplit, long split_stride, long cols, int col0, int C,
    const float* __restrict__ in_bias, float* __restrict__ state, long slot_stride, int taps,
    const int* __restrict__ slots, const int* __restrict__ span_start, const int* __restrict__ span_pos) {
  const int c = blockIdx.x * kRecThreads + threadIdx.x;
  if (c >= C) return;
  const int span = blockIdx.y;
  const int K = taps - 1;
  const long t0 = span_start[span], t1 = span_start[span + 1];
  const long len = t1 - t0;
  const bool fresh = span_pos[span] == 0;
  float* st = state + (long)slots[span] * slot_stride + (long)c * K;
  float old[kMaxTaps];
  for (int j = 0; j < K; ++j) old[j] = fresh ? 0.f : st[j];
  for (int j = 0; j < K; ++j) {
    const long row = t1 - K + j;
    st[j] = row >= t0 ? conv_input(proj, nsplit, split_stride, cols, col0 + c, in_bias, row) : old[j + len];
  }
}

// ---------------------------------------------------------------------------- gated delta rule

// proj: [nsplit][n][cols], columns q (G*dk) | k (G*dk) | v (H*dv) | b (H) | a (H) | gate (H*dv) |
// whatever else the product made.  With `a_sums` ([a_ns][n][a_row], the first H*dk of a row) the
// decay has one number per head and key channel, from sums of their own, and proj has no a
// columns; with `gate_sums` ([g_ns][n][g_row], the first H*dv of a row) the gate's sums are their
// own too and proj has no gate columns.
// One wave per (token, item): the items are the G query heads, the G key heads and the H value
// heads; a value head's wave also makes that head's gate, decays and beta.  A lane keeps up to
// four channels of a query or key head (heads of up to 256) between the sum and the division.
__global__ __launch_bounds__(kRecThreads) void gated_delta_prep_kernel(
    const float* __restrict__ proj, int nsplit, long split_stride, const float* __restrict__ conv_w, int taps,
    const float* __restrict__ state, long slot_stride, const float* __restrict__ a_log,
    const float* __restrict__ dt_bias, const int* __restrict__ span_of_token, const int* __restrict__ slots,
    const int* __restrict__ span_start, const int* __restrict__ span_pos, float* __restrict__ qn,
    float* __restrict__ kn, float* __restrict__ vv, float* __restrict__ gb, float* __restrict__ gate, int H, int G,
    int dk, int dv, float unit_eps, long cols, const float* __restrict__ a_sums, int a_ns, long a_stride, long a_row,
    const float* __restrict__ gate_sums, int g_ns, long g_stride, long g_row, int gate_sigmoid,
    float* __restrict__ dec) {
  const long t = blockIdx.x;
  const int lane = threadIdx.x % kWave;
  const int item = blockIdx.y * (kRecThreads / kWave) + threadIdx.x / kWave;
  if (item >= 2 * G + H) return;
  const int QK = G * dk, HV = H * dv, C = 2 * QK + HV;
  const int gate_col = C + (a_sums ? H : 2 * H);
  const int span = span_of_token[t];
  const long t0 = span_start[span];
  const bool fresh = span_pos[span] == 0;
  const float* st = state + (long)slots[span] * slot_stride;
  auto convolved = [&](int c) {
    const float y = conv_at(proj, nsplit, split_stride, cols, c, nullptr, conv_w + (long)c * taps, taps,
                            st + (long)c * (taps - 1), fresh, t, t0);
    return y / (1.f + expf(-y));                         // SiLU
  };
  if (item < 2 * G) {        // a head of q or k: the unit norm
    const int c0 = item * dk;                            // q's heads, then k's, lie side by side
    float val[4];
    float ss = 0.f;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int e = lane + kWave * r;
      val[r] = e < dk ? convolved(c0 + e) : 0.f;
      ss = fmaf(val[r], val[r], ss);
    }
    ss = wave_sum(ss);
    const bool is_q = item < G;
    const float f = (is_q ? 1.f / sqrtf((float)dk) : 1.f) / sqrtf(ss + unit_eps);
    float* dst = is_q ? qn + t * QK + (long)item * dk : kn + t * QK + (long)(item - G) * dk;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int e = lane + kWave * r;
      if (e < dk) dst[e] = val[r] * f;
    }
    return;
  }
  const int h = item - 2 * G;
  for (int e = lane; e < dv; e += kWave) {
    const int c = h * dv + e;
    vv[t * HV + c] = convolved(2 * QK + c);
    float g = 0.f;
    if (gate_sums)
      for (int s = 0; s < g_ns; ++s) g += gate_sums[s * g_stride + t * g_row + c];
    else
      for (int s = 0; s < nsplit; ++s) g += proj[s * split_stride + t * cols + gate_col + c];
    gate[t * HV + c] = gate_sigmoid ? sigmoid_f32(g) : g / (1.f + expf(-g));
  }
  if (a_sums) {       // one decay per head and key channel; dt_bias has as many entries
    const float rate = expf(a_log[h]);
    for (int e = lane; e < dk; e += kWave) {
      const int c = h * dk + e;
      float a = 0.f;
      for (int s = 0; s < a_ns; ++s) a += a_sums[s * a_stride + t * a_row + c];
      dec[t * (long)H * dk + c] = expf(-rate * softplus_f32(a + dt_bias[c]));
    }
  }
  if (lane == 0) {
    float b = 0.f, a = 0.f;
    for (int s = 0; s < nsplit; ++s) {
      b += proj[s * split_stride + t * cols + C + h];
      if (!a_sums) a += proj[s * split_stride + t * cols + C + H + h];
    }
    gb[t * 2 * H + h] = a_sums ? 1.f : expf(-expf(a_log[h]) * softplus_f32(a + dt_bias[h]));
    gb[t * 2 * H + H + h] = sigmoid_f32(b);
  }
}

constexpr int kDeltaParts = 16;                              // lanes that share a column of the state
constexpr int kDeltaCols = kRecThreads / kDeltaParts;        // columns of a workgroup
constexpr int kDeltaBlock = 16;                              // tokens staged at a time

// Thread (j, p): column j of the workgroup's block of value channels, rows p, p + 16, ... of it.
// A block of tokens' vectors goes through LDS: k and q [TB][dk] each, v [TB][16 columns], g and
// beta [TB]; the sums over a column's rows are lane exchanges within its sixteen lanes.
// VEC: the decay has one number per head and key channel (`dec` [n][H*dk], staged like the keys)
// instead of one per head.
template <int NR, bool VEC>
__global__ __launch_bounds__(kRecThreads) void gated_delta_scan_kernel(
    const float* __restrict__ qn, const float* __restrict__ kn, const float* __restrict__ vv,
    const float* __restrict__ gb, float* __restrict__ o_out, float* __restrict__ state, long slot_stride,
    const int* __restrict__ slots, const int* __restrict__ span_start, const int* __restrict__ span_pos, int H, int G,
    int dk, int dv, const float* __restrict__ dec) {
  extern __shared__ float lds[];
  float* ks = lds;                                   // [TB][dk]
  float* qs = ks + kDeltaBlock * dk;                 // [TB][dk]
  float* vs = qs + kDeltaBlock * dk;                 // [TB][kDeltaCols]
  float* gs = vs + kDeltaBlock * kDeltaCols;         // [TB][2]
  float* ds = gs + 2 * kDeltaBlock;                  // [TB][dk] (VEC)
  const int span = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int g = h / (H / G);
  const int jl = tid / kDeltaParts, p = tid % kDeltaParts;
  const int j = blockIdx.z * kDeltaCols + jl;
  const bool col = j < dv;
  const long t0 = span_start[span], t1 = span_start[span + 1];
  const bool fresh = span_pos[span] == 0;
  float* S = state + (long)slots[span] * slot_stride + (long)h * dk * dv;
  float s[NR];
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int r = p + kDeltaParts * i;
    s[i] = (col && r < dk && !fresh) ? S[(long)r * dv + j] : 0.f;
  }
  const int QK = G * dk, HV = H * dv;
  // A thread's pieces of a block of tokens: NR elements of k and of q (element i = tid + 256 j of
  // [TB][dk]), one of v, one of g and beta.  They are asked for one block ahead and wait in
  // registers while the block before them is multiplied.
  int tt_of[NR], e_of[NR];
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int idx = tid + kRecThreads * i;
    tt_of[i] = idx < kDeltaBlock * dk ? idx / dk : kDeltaBlock;      // kDeltaBlock: no such element
    e_of[i] = idx - tt_of[i] * dk;
  }
  const int v_tt = tid / kDeltaCols, v_c = blockIdx.z * kDeltaCols + tid % kDeltaCols;
  struct Pieces {
    float k[NR], q[NR], d[VEC ? NR : 1], v, g;
  };
  auto fetch = [&](long tb, int nt) -> Pieces {
    Pieces P;
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const bool ok = tt_of[i] < nt;
      const long at = (tb + (ok ? tt_of[i] : 0)) * QK + (long)g * dk + (ok ? e_of[i] : 0);
      P.k[i] = ok ? kn[at] : 0.f;
      P.q[i] = ok ? qn[at] : 0.f;
      if constexpr (VEC)
        P.d[i] = ok ? dec[(tb + tt_of[i]) * (long)H * dk + (long)h * dk + e_of[i]] : 0.f;
    }
    P.v = (v_tt < nt && v_c < dv) ? vv[(tb + v_tt) * HV + (long)h * dv + v_c] : 0.f;
    P.g = tid < 2 * nt ? gb[(tb + tid / 2) * 2 * H + (tid % 2) * H + h] : 0.f;
    return P;
  };
  long tb = t0;
  int nt = (int)min((long)kDeltaBlock, t1 - tb);
  Pieces pre = fetch(tb, nt);
  while (tb < t1) {
    __syncthreads();                                 // the block before this one has been read
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int idx = tid + kRecThreads * i;
      if (idx < kDeltaBlock * dk) {
        ks[idx] = pre.k[i];
        qs[idx] = pre.q[i];
        if constexpr (VEC) ds[idx] = pre.d[i];
      }
    }
    vs[tid] = pre.v;                                 // [TB][kDeltaCols]: kRecThreads elements
    if (tid < 2 * kDeltaBlock) gs[tid] = pre.g;
    __syncthreads();
    const long tb_next = tb + kDeltaBlock;
    const int nt_next = (int)max(0L, min((long)kDeltaBlock, t1 - tb_next));
    if (nt_next > 0) pre = fetch(tb_next, nt_next);
    for (int tt = 0; tt < nt; ++tt) {
      const float decay = gs[2 * tt], beta = gs[2 * tt + 1];
      const float* kt = ks + tt * dk;
      const float* qt = qs + tt * dk;
      float kr[NR], dot = 0.f;
#pragma unroll
      for (int i = 0; i < NR; ++i) {
        const int r = p + kDeltaParts * i;
        kr[i] = r < dk ? kt[r] : 0.f;
        if constexpr (VEC) s[i] *= r < dk ? ds[tt * dk + r] : 0.f; else s[i] *= decay;
        dot = fmaf(s[i], kr[i], dot);
      }
      dot = parts_sum<kDeltaParts>(dot);
      const float u = beta * (vs[tt * kDeltaCols + jl] - dot);
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < NR; ++i) {
        const int r = p + kDeltaParts * i;
        s[i] = fmaf(kr[i], u, s[i]);
        o = fmaf(s[i], r < dk ? qt[r] : 0.f, o);
      }
      o = parts_sum<kDeltaParts>(o);
      if (col && p == 0) o_out[(tb + tt) * HV + (long)h * dv + j] = o;
    }
    tb = tb_next;
    nt = nt_next;
  }
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int r = p + kDeltaParts * i;
    if (col && r < dk) S[(long)r * dv + j] = s[i];
  }
}

// ---------------------------------------------------------------------------- gated linear recurrence

constexpr int kGateTokens = 8;       // tokens of a tile of the gates' products
constexpr int kGateOuts = kRecThreads / 4;   // output channels of a workgroup

// proj: [nsplit][n][2 W], columns y | x.  Workgroup (tile of tokens, block b of the gates, 64 of
// its output channels): the convolved inputs of the block's channels for the tile's tokens go
// into LDS [TT][bs]; the gates' matrices are read [block][in][out] so that neighbouring threads
// read neighbouring weights.
__global__ __launch_bounds__(kRecThreads) void linear_recurrence_prep_kernel(
    const float* __restrict__ proj, int nsplit, long split_stride, const float* __restrict__ x_bias,
    const float* __restrict__ conv_w, const float* __restrict__ conv_b, int taps, const float* __restrict__ state,
    long slot_stride, const float* __restrict__ wr_t, const float* __restrict__ wi_t, const float* __restrict__ br,
    const float* __restrict__ bi, const float* __restrict__ rate, const int* __restrict__ span_of_token,
    const int* __restrict__ slots, const int* __restrict__ span_start, const int* __restrict__ span_pos,
    float* __restrict__ a_out, float* __restrict__ b_out, int n, int W, int bs) {
  extern __shared__ float us[];                      // [TT][bs]
  const int tile = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
  const long tfirst = (long)tile * kGateTokens;
  const int nt = (int)min((long)kGateTokens, n - tfirst);
  const long cols = 2L * W;
  for (int i = tid; i < nt * bs; i += kRecThreads) {
    const int tt = i / bs, c = b * bs + i % bs;
    const long t = tfirst + tt;
    const int span = span_of_token[t];
    // (the convolution's input carries the projection's bias; before position 0 it is zero)
    us[i] = conv_at(proj, nsplit, split_stride, cols, W + c, x_bias - W, conv_w + (long)c * taps, taps,
                    state + (long)slots[span] * slot_stride + (long)c * (taps - 1), span_pos[span] == 0, t,
                    span_start[span]) + conv_b[c];
  }
  for (int i = nt * bs + tid; i < kGateTokens * bs; i += kRecThreads) us[i] = 0.f;
  __syncthreads();
  const float* wr = wr_t + (long)b * bs * bs;
  const float* wi = wi_t + (long)b * bs * bs;
  // A workgroup takes kGateOuts output channels (blockIdx.z); four threads share an output, a
  // quarter of the inputs each, and meet in LDS: a chain of bs / 4 multiply-adds, and four times
  // the workgroups, where a decode step has one tile of tokens.
  __shared__ float red[3][kGateOuts][2 * kGateTokens];
  const int ol = tid % kGateOuts, part = tid / kGateOuts;
  const int o = blockIdx.z * kGateOuts + ol;
  const bool o_ok = o < bs;
  const int per = (bs + 3) / 4, i0 = part * per, i1 = min(bs, i0 + per);
  float ar[kGateTokens], ai[kGateTokens];
#pragma unroll
  for (int tt = 0; tt < kGateTokens; ++tt) ar[tt] = ai[tt] = 0.f;
  if (o_ok) {
#pragma unroll 4
    for (int i = i0; i < i1; ++i) {
      const float r = wr[(long)i * bs + o], g = wi[(long)i * bs + o];
#pragma unroll
      for (int tt = 0; tt < kGateTokens; ++tt) {
        const float u = us[tt * bs + i];
        ar[tt] = fmaf(r, u, ar[tt]);
        ai[tt] = fmaf(g, u, ai[tt]);
      }
    }
  }
  if (part > 0) {
#pragma unroll
    for (int tt = 0; tt < kGateTokens; ++tt) {
      red[part - 1][ol][2 * tt] = ar[tt];
      red[part - 1][ol][2 * tt + 1] = ai[tt];
    }
  }
  __syncthreads();
  if (part > 0 || !o_ok) return;
#pragma unroll
  for (int q = 0; q < 3; ++q)          // in a fixed order
#pragma unroll
    for (int tt = 0; tt < kGateTokens; ++tt) {
      ar[tt] += red[q][ol][2 * tt];
      ai[tt] += red[q][ol][2 * tt + 1];
    }
  const int c = b * bs + o;
  const float rb = br[c], ib = bi[c], rt = rate[c];
#pragma unroll
  for (int tt = 0; tt < kGateTokens; ++tt) {
    if (tt >= nt) break;
    const float r = sigmoid_f32(ar[tt] + rb), ig = sigmoid_f32(ai[tt] + ib);
    const float log_a = -rt * r;
    const float a = expf(log_a);
    const float mult = sqrtf(fmaxf(-expm1f(2.f * log_a), 0.f));      // sqrt(1 - a^2)
    a_out[(tfirst + tt) * W + c] = a;
    b_out[(tfirst + tt) * W + c] = mult * ig * us[tt * bs + o];
  }
}

// S <- a S + b along a span; out = S * gelu_tanh(y + y_bias).  Eight tokens' numbers are asked
// for at a time, so that the chain holds arithmetic only.
// A span's tokens are cut into kScanSegs segments, one wave each (64 channels a workgroup):
// S_t = a_t S_(t-1) + b_t is a composition of maps S -> a S + b, and so is a whole segment's
// (A S + B, with A the product of its a and B its own chain from zero).  Every wave first runs its
// segment's chain from zero, the segments' (A, B) meet in LDS, a wave folds those before its own
// into its starting state and runs its segment once more, now writing.  A chain of n steps
// becomes two of n / kScanSegs.
constexpr int kScanCh = 64;
constexpr int kScanSegs = 16;

template <typename T>
__global__ __launch_bounds__(kScanCh * kScanSegs) void linear_recurrence_scan_kernel(
    const float* __restrict__ a_in, const float* __restrict__ b_in, const float* __restrict__ proj, int nsplit,
    long split_stride, const float* __restrict__ y_bias, float* __restrict__ state, long slot_stride,
    const int* __restrict__ slots, const int* __restrict__ span_start, const int* __restrict__ span_pos,
    T* __restrict__ out, int W) {
  __shared__ float seg_a[kScanSegs][kScanCh], seg_b[kScanSegs][kScanCh];
  const int lane = threadIdx.x % kScanCh, seg = threadIdx.x / kScanCh;
  const int c = min((int)blockIdx.x * kScanCh + lane, W - 1);
  const bool ok = blockIdx.x * kScanCh + lane < W;
  const int span = blockIdx.y;
  const long t0 = span_start[span], t1 = span_start[span + 1];
  const long per = (t1 - t0 + kScanSegs - 1) / kScanSegs;
  const long a0 = min(t1, t0 + seg * per), a1 = min(t1, a0 + per);
  constexpr int U = 8;
  float A = 1.f, B = 0.f;
  {
    for (long tb = a0; tb < a1; tb += U) {
      float a[U], b[U];
#pragma unroll
      for (int q = 0; q < U; ++q) {
        const long t = min(tb + q, a1 - 1);
        a[q] = a_in[t * W + c];
        b[q] = b_in[t * W + c];
      }
#pragma unroll
      for (int q = 0; q < U; ++q) {
        if (tb + q >= a1) break;
        B = fmaf(a[q], B, b[q]);
        A *= a[q];
      }
    }
  }
  seg_a[seg][lane] = A;
  seg_b[seg][lane] = B;
  __syncthreads();
  float* st = state + (long)slots[span] * slot_stride + c;
  float S = span_pos[span] == 0 ? 0.f : *st;
  for (int s = 0; s < seg; ++s) S = fmaf(seg_a[s][lane], S, seg_b[s][lane]);
  const float yb = y_bias[c];
  for (long tb = a0; tb < a1; tb += U) {
    float a[U], b[U], y[U];
#pragma unroll
    for (int q = 0; q < U; ++q) {
      const long t = min(tb + q, a1 - 1);
      a[q] = a_in[t * W + c];
      b[q] = b_in[t * W + c];
      float v = 0.f;
      for (int s = 0; s < nsplit; ++s) v += proj[s * split_stride + t * 2 * W + c];
      y[q] = gate_act(v + yb, ACT_GELU_TANH);
    }
#pragma unroll
    for (int q = 0; q < U; ++q) {
      if (tb + q >= a1) break;
      S = fmaf(a[q], S, b[q]);
      if (ok) out[(tb + q) * W + c] = from_f32<T>(S * y[q]);
    }
  }
  // the wave of the last segment ends at the span's last token (an empty segment has folded all)
  if (ok && seg == kScanSegs - 1) *st = S;
}

// out = sa * (sum of a's slices) + sb * (sum of b's slices), element by element.
__global__ void scaled_sum_kernel(float* __restrict__ out, const float* __restrict__ a, int na, long stride_a, float sa,
                                  const float* __restrict__ b, int nb, long stride_b, float sb, long count) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count) return;
  float va = 0.f, vb = 0.f;
  for (int s = 0; s < na; ++s) va += a[i + s * stride_a];
  for (int s = 0; s < nb; ++s) vb += b[i + s * stride_b];
  out[i] = fmaf(sa, va, sb * vb);
}

// out = sa * wa * N(sum of a's slices) + sb * wb * N(sum of b's slices), row by row; N(v) = v /
// sqrt(mean(v^2) + eps).  One workgroup a row; both rows wait in LDS between the two passes.
__global__ __launch_bounds__(kRecThreads) void normed_sum_kernel(
    float* __restrict__ out, const float* __restrict__ a, int na, long stride_a, float sa, const float* __restrict__ wa,
    const float* __restrict__ b, int nb, long stride_b, float sb, const float* __restrict__ wb, int d, float eps) {
  extern __shared__ float rows_lds[];     // [2][d]
  __shared__ float red[16];
  const long r = blockIdx.x;
  float ssa = 0.f, ssb = 0.f;
  for (int i = threadIdx.x; i < d; i += kRecThreads) {
    float va = 0.f, vb = 0.f;
    for (int s = 0; s < na; ++s) va += a[r * d + i + s * stride_a];
    for (int s = 0; s < nb; ++s) vb += b[r * d + i + s * stride_b];
    rows_lds[i] = va;
    rows_lds[d + i] = vb;
    ssa = fmaf(va, va, ssa);
    ssb = fmaf(vb, vb, ssb);
  }
  const float ra = sa / sqrtf(block_sum(ssa, red) / (float)d + eps);
  const float rb = sb / sqrtf(block_sum(ssb, red) / (float)d + eps);
  for (int i = threadIdx.x; i < d; i += kRecThreads)     // a thread reads back what it wrote itself
    out[r * d + i] = fmaf(rows_lds[i] * ra, wa[i], rows_lds[d + i] * rb * wb[i]);
}

}  // namespace kllm

using namespace kllm;

extern "C" int kllm_normed_sum(float* out, const float* a, int na, long stride_a, float sa, const float* wa,
                               const float* b, int nb, long stride_b, float sb, const float* wb, int n, int d,
                               float eps, hipStream_t stream) {
  KLLM_REQUIRE(out && a && b && wa && wb && na >= 1 && nb >= 1 && n > 0 && d > 0, "normed_sum: null pointer or bad sizes");
  const size_t lds = 2 * (size_t)d * sizeof(float);
  KLLM_REQUIRE(lds <= 128 * 1024, "normed_sum: rows of %d do not fit into LDS", d);
  static size_t raised_to = 48 * 1024;
  if (lds > raised_to) {
    (void)hipFuncSetAttribute((const void*)normed_sum_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    raised_to = lds;
  }
  hipLaunchKernelGGL(normed_sum_kernel, dim3(n), dim3(kRecThreads), lds, stream, out, a, na, stride_a, sa, wa, b, nb,
                     stride_b, sb, wb, d, eps);
  KLLM_CHECK_LAUNCH("normed_sum");
  return 0;
}

extern "C" int kllm_scaled_sum(float* out, const float* a, int na, long stride_a, float sa, const float* b, int nb,
                               long stride_b, float sb, long count, hipStream_t stream) {
  KLLM_REQUIRE(out && a && b && na >= 1 && nb >= 1 && count > 0, "scaled_sum: null pointer or bad sizes");
  hipLaunchKernelGGL(scaled_sum_kernel, dim3(ceil_div(count, 256)), dim3(256), 0, stream, out, a, na, stride_a, sa, b, nb,
                     stride_b, sb, count);
  KLLM_CHECK_LAUNCH("scaled_sum");
  return 0;
}

extern "C" int kllm_conv_state_update(const float* proj, int nsplit, long split_stride, int cols, int col0, int C,
                                      const float* in_bias, float* state, long slot_stride, int taps, const int* slots,
                                      const int* span_start, const int* span_pos, int n_spans, hipStream_t stream) {
  KLLM_REQUIRE(proj && state && slots && span_start && span_pos, "conv_state_update: null pointer");
  KLLM_REQUIRE(nsplit >= 1 && cols > 0 && col0 >= 0 && C > 0 && col0 + C <= cols && n_spans > 0 && n_spans <= 65535,
               "conv_state_update: bad sizes cols=%d col0=%d C=%d spans=%d", cols, col0, C, n_spans);
  KLLM_REQUIRE(taps >= 1 && taps <= kMaxTaps, "conv_state_update: %d taps (1 to %d)", taps, kMaxTaps);
  if (taps == 1) return 0;
  hipLaunchKernelGGL(conv_state_update_kernel, dim3(ceil_div(C, kRecThreads), n_spans), dim3(kRecThreads), 0, stream,
                     proj, nsplit, split_stride, (long)cols, col0, C, in_bias ? in_bias - col0 : nullptr, state,
                     slot_stride, taps, slots, span_start, span_pos);
  KLLM_CHECK_LAUNCH("conv_state_update");
  return 0;
}

extern "C" int kllm_gated_delta_prep(const float* proj, int nsplit, long split_stride, const float* conv_w, int taps,
                                     const float* state, long slot_stride, const float* a_log, const float* dt_bias,
                                     const int* span_of_token, const int* slots, const int* span_start,
                                     const int* span_pos, float* qn, float* kn, float* vv, float* gb, float* gate,
                                     int n, int H, int G, int dk, int dv, float unit_eps, int cols,
                                     const float* a_sums, int a_ns, long a_stride, int a_row, const float* gate_sums,
                                     int g_ns, long g_stride, int g_row, int gate_sigmoid, float* dec,
                                     hipStream_t stream) {
  KLLM_REQUIRE(proj && conv_w && state && a_log && dt_bias && span_of_token && slots && span_start && span_pos && qn &&
                   kn && vv && gb && gate, "gated_delta_prep: null pointer");
  KLLM_REQUIRE((a_sums == nullptr) == (dec == nullptr) && (!a_sums || a_ns >= 1) && (!gate_sums || g_ns >= 1),
               "gated_delta_prep: decays per key channel come with their sums and a place for them");
  KLLM_REQUIRE(cols >= 2 * G * dk + H * dv + (a_sums ? H : 2 * H) + (gate_sums ? 0 : H * dv),
               "gated_delta_prep: %d columns do not hold the projections", cols);
  KLLM_REQUIRE(n > 0 && H > 0 && G > 0 && H % G == 0 && dk > 0 && dv > 0 && nsplit >= 1,
               "gated_delta_prep: bad sizes n=%d H=%d G=%d dk=%d dv=%d", n, H, G, dk, dv);
  KLLM_REQUIRE(taps >= 1 && taps <= kMaxTaps, "gated_delta_prep: %d taps (1 to %d)", taps, kMaxTaps);
  KLLM_REQUIRE(dk <= 4 * kWave, "gated_delta_prep: key heads of %d (up to %d)", dk, 4 * kWave);
  KLLM_REQUIRE((!a_sums || a_row >= H * dk) && (!gate_sums || g_row >= H * dv),
               "gated_delta_prep: rows of %d and %d sums do not hold the decays and the gates", a_row, g_row);
  const int items = 2 * G + H, per_wg = kRecThreads / kWave;
  KLLM_REQUIRE(ceil_div(items, per_wg) <= 65535, "gated_delta_prep: %d heads are too many for the grid", items);
  hipLaunchKernelGGL(gated_delta_prep_kernel, dim3(n, ceil_div(items, per_wg)), dim3(kRecThreads), 0, stream, proj,
                     nsplit, split_stride, conv_w, taps, state, slot_stride, a_log, dt_bias, span_of_token, slots,
                     span_start, span_pos, qn, kn, vv, gb, gate, H, G, dk, dv, unit_eps, (long)cols, a_sums, a_ns,
                     a_stride, (long)a_row, gate_sums, g_ns, g_stride, (long)g_row, gate_sigmoid, dec);
  KLLM_CHECK_LAUNCH("gated_delta_prep");
  return 0;
}

extern "C" int kllm_gated_delta_max_dim(void) { return 16 * kDeltaParts; }

extern "C" int kllm_gated_delta_scan(const float* qn, const float* kn, const float* vv, const float* gb, float* o_out,
                                     float* state, long slot_stride, const int* slots, const int* span_start,
                                     const int* span_pos, int n_spans, int H, int G, int dk, int dv, const float* dec,
                                     hipStream_t stream) {
  KLLM_REQUIRE(qn && kn && vv && gb && o_out && state && slots && span_start && span_pos,
               "gated_delta_scan: null pointer");
  KLLM_REQUIRE(n_spans > 0 && H > 0 && H <= 65535 && G > 0 && H % G == 0 && dk > 0 && dk <= 16 * kDeltaParts && dv > 0,
               "gated_delta_scan: bad sizes spans=%d H=%d G=%d dk=%d dv=%d (keys of up to %d)", n_spans, H, G, dk, dv,
               16 * kDeltaParts);
  const dim3 grid(n_spans, H, ceil_div(dv, kDeltaCols));
  KLLM_REQUIRE(grid.z <= 65535, "gated_delta_scan: values too wide for the grid");
  const size_t lds = ((size_t)kDeltaBlock * ((dec ? 3 : 2) * dk + kDeltaCols + 2)) * sizeof(float);
  const int nr = ceil_div(dk, kDeltaParts);
#define KLLM_GDS(NR)                                                                                                   \
  do {                                                                                                                 \
    if (dec)                                                                                                           \
      hipLaunchKernelGGL((gated_delta_scan_kernel<NR, true>), grid, dim3(kRecThreads), lds, stream, qn, kn, vv, gb,    \
                         o_out, state, slot_stride, slots, span_start, span_pos, H, G, dk, dv, dec);                   \
    else                                                                                                               \
      hipLaunchKernelGGL((gated_delta_scan_kernel<NR, false>), grid, dim3(kRecThreads), lds, stream, qn, kn, vv, gb,   \
                         o_out, state, slot_stride, slots, span_start, span_pos, H, G, dk, dv, dec);                   \
  } while (0)
  if (nr <= 1) KLLM_GDS(1);
  else if (nr <= 2) KLLM_GDS(2);
  else if (nr <= 4) KLLM_GDS(4);
  else if (nr <= 8) KLLM_GDS(8);
  else KLLM_GDS(16);
#undef KLLM_GDS
  KLLM_CHECK_LAUNCH("gated_delta_scan");
  return 0;
}

extern "C" int kllm_linear_recurrence_prep(const float* proj, int nsplit, long split_stride, const float* x_bias,
                                           const float* conv_w, const float* conv_b, int taps, const float* state,
                                           long slot_stride, const float* wr_t, const float* wi_t, const float* br,
                                           const float* bi, const float* rate, const int* span_of_token,
                                           const int* slots, const int* span_start, const int* span_pos, float* a_out,
                                           float* b_out, int n, int W, int blocks, hipStream_t stream) {
  KLLM_REQUIRE(proj && x_bias && conv_w && conv_b && state && wr_t && wi_t && br && bi && rate && span_of_token &&
                   slots && span_start && span_pos && a_out && b_out, "linear_recurrence_prep: null pointer");
  KLLM_REQUIRE(n > 0 && W > 0 && blocks > 0 && blocks <= 65535 && W % blocks == 0 && nsplit >= 1,
               "linear_recurrence_prep: bad sizes n=%d W=%d blocks=%d", n, W, blocks);
  KLLM_REQUIRE(taps >= 1 && taps <= kMaxTaps, "linear_recurrence_prep: %d taps (1 to %d)", taps, kMaxTaps);
  const int bs = W / blocks;
  const size_t lds = (size_t)kGateTokens * bs * sizeof(float);
  KLLM_REQUIRE(lds <= 128 * 1024, "linear_recurrence_prep: blocks of %d channels do not fit into LDS", bs);
  static size_t raised_to = 48 * 1024;      // beside the kernel's own 12 KB
  if (lds > raised_to) {
    (void)hipFuncSetAttribute((const void*)linear_recurrence_prep_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    raised_to = lds;
  }
  hipLaunchKernelGGL(linear_recurrence_prep_kernel, dim3(ceil_div(n, kGateTokens), blocks, ceil_div(bs, kGateOuts)), dim3(kRecThreads), lds,
                     stream, proj, nsplit, split_stride, x_bias, conv_w, conv_b, taps, state, slot_stride, wr_t, wi_t,
                     br, bi, rate, span_of_token, slots, span_start, span_pos, a_out, b_out, n, W, bs);
  KLLM_CHECK_LAUNCH("linear_recurrence_prep");
  return 0;
}

extern "C" int kllm_linear_recurrence_scan(const float* a_in, const float* b_in, const float* proj, int nsplit,
                                           long split_stride, const float* y_bias, float* state, long slot_stride,
                                           const int* slots, const int* span_start, const int* span_pos, void* out,
                                           int n_spans, int W, int dtype, hipStream_t stream) {
  KLLM_REQUIRE(a_in && b_in && proj && y_bias && state && slots && span_start && span_pos && out,
               "linear_recurrence_scan: null pointer");
  KLLM_REQUIRE(n_spans > 0 && n_spans <= 65535 && W > 0 && nsplit >= 1, "linear_recurrence_scan: bad sizes spans=%d W=%d",
               n_spans, W);
  KLLM_REQUIRE(dtype == DT_F32 || dtype == DT_BF16, "linear_recurrence_scan: unknown dtype %d", dtype);
  const dim3 grid(ceil_div(W, kScanCh), n_spans);
  if (dtype == DT_F32)
    hipLaunchKernelGGL(linear_recurrence_scan_kernel<float>, grid, dim3(kScanCh * kScanSegs), 0, stream, a_in, b_in, proj,
                       nsplit, split_stride, y_bias, state, slot_stride, slots, span_start, span_pos, (float*)out, W);
  else
    hipLaunchKernelGGL(linear_recurrence_scan_kernel<bf16_t>, grid, dim3(kScanCh * kScanSegs), 0, stream, a_in, b_in, proj,
                       nsplit, split_stride, y_bias, state, slot_stride, slots, span_start, span_pos, (bf16_t*)out, W);
  KLLM_CHECK_LAUNCH("linear_recurrence_scan");
  return 0;
}
