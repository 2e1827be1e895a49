// A routed feed-forward (mixture of experts) whose launches depend on the step's shape only:
// which token goes to which expert stays on the device.
//
//   kllm_moe_route    per token: softmax (or the logistic function) of the router's sums over all
//                     experts, the `top` largest of (score + correction), optionally only among
//                     the experts of the best groups of neighbours, their scores divided by their
//                     sum (or not) and times a constant; a shared expert's gate from one more sum
//   kllm_moe_plan     the (token, choice) entries grouped by expert, and a list of tiles of up to
//                     64 entries of one expert (a fixed number of tiles, the unused ones empty)
//   kllm_moe_expert   one tile's product with its expert's weights on the matrix cores (64 rows by
//                     64 columns a workgroup through LDS, or 128 by 128; 32-bit or bfloat16
//                     operands): gate and up with the gate in the epilogue, or down
//   kllm_moe_expert_rows  the same products entry by entry, for decode batches: no plan, a wave
//                     per two columns, the whole of K of a row in flight at once
//   kllm_moe_combine  per token the weighted sum of its choices' outputs, in the order of the
//                     choices; an expert beyond the last real one is the identity (its output is
//                     the feed-forward's input); plus the sums of a shared expert
//
// A row's result depends on the row alone: on no other entry of its tile and not on where in
// the tile it lies.
#include <math.h>

#include "common.hpp"
#include "kllm_kernels.h"

namespace kllm {

constexpr int kMoeTileRows = 64;     // rows of the small tiles; the large ones have twice as many
constexpr int kMaxTop = 128;        // experts a token may use at most
constexpr int kMaxRouted = 4096;    // experts a router may choose from at most

// One wave per token; a lane takes the experts lane, lane + 64, ...  The largest of a set is
// found lane by lane and then across the wave, the lower expert winning a tie.
// scoring 0: s = softmax(z); 1: s = 1 / (1 + exp(-z)).  groups > 1: the experts form `groups` equal
// groups of neighbours, a group's score is the sum of its two largest s + correction, and only
// experts of the `keep` best groups (the lower group winning a tie) can be chosen; lane g works
// out group g's score.  The weights are the chosen s times `scale`, divided by their sum first
// if `renorm`.  z's rows are `cols` sums long; with `sgate` the sum behind the experts' is a
// gate's: sgate[t] = 1 / (1 + exp(-z[t][R])).
__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ z, int nsplit, long split_stride,
                                                        const float* __restrict__ correction, int n, int R, int top,
                                                        int* __restrict__ idx, float* __restrict__ wgt, int scoring,
                                                        int groups, int keep, float scale, int renorm, int cols,
                                                        float* __restrict__ sgate) {
  const int t = blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  if (t >= n) return;
  auto z_at = [&](int e) {
    float v = 0.f;
    for (int s = 0; s < nsplit; ++s) v += z[s * split_stride + (long)t * cols + e];
    return v;
  };
  float m = 0.f, den = 1.f;
  if (scoring == 0) {
    m = -INFINITY;
    for (int e = lane; e < R; e += kWave) m = fmaxf(m, z_at(e));
    m = wave_max(m);
    den = 0.f;
    for (int e = lane; e < R; e += kWave) den += expf(z_at(e) - m);
    den = wave_sum(den);
  }
  auto score_at = [&](int e) { return scoring == 0 ? expf(z_at(e) - m) / den : 1.f / (1.f + expf(-z_at(e))); };
  if (sgate && lane == 0) sgate[t] = 1.f / (1.f + expf(-z_at(R)));
  unsigned long long open_groups = ~0ull;      // bit g: experts of group g can be chosen
  const int gsize = R / (groups > 1 ? groups : 1);
  if (groups > 1) {
    float gscore = -INFINITY;
    if (lane < groups) {
      float a = -INFINITY, b = -INFINITY;      // the two largest of the group
      for (int e = lane * gsize; e < (lane + 1) * gsize; ++e) {
        const float c = correction ? score_at(e) + correction[e] : score_at(e);
        if (c > a) {
          b = a;
          a = c;
        } else if (c > b) {
          b = c;
        }
      }
      gscore = gsize > 1 ? a + b : a;
    }
    open_groups = 0;
    for (int k = 0; k < keep; ++k) {
      float best = gscore;
      int who = lane;
#pragma unroll
      for (int off = kWave / 2; off > 0; off >>= 1) {
        const float ob = __shfl_xor(best, off, kWave);
        const int ow = __shfl_xor(who, off, kWave);
        if (ob > best || (ob == best && ow < who)) {
          best = ob;
          who = ow;
        }
      }
      open_groups |= 1ull << who;
      if (lane == who) gscore = -INFINITY;
    }
  }
  float picked = 0.f;
  float mine[kMaxTop / kWave] = {};
  unsigned long long taken = 0;      // bit i: this lane's expert lane + 64 i is chosen already
  for (int k = 0; k < top; ++k) {
    int best = R;
    float best_choice = -INFINITY, best_score = 0.f;
    for (int e = lane; e < R; e += kWave) {
      if ((taken >> (e / kWave)) & 1) continue;
      if (groups > 1 && !((open_groups >> (e / gsize)) & 1)) continue;
      const float s = score_at(e);
      const float c = correction ? s + correction[e] : s;
      if (c > best_choice) {
        best_choice = c;
        best_score = s;
        best = e;
      }
    }
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
      const float oc = __shfl_xor(best_choice, off, kWave), os = __shfl_xor(best_score, off, kWave);
      const int ob = __shfl_xor(best, off, kWave);
      if (oc > best_choice || (oc == best_choice && ob < best)) {
        best_choice = oc;
        best_score = os;
        best = ob;
      }
    }
    if (best % kWave == lane) taken |= 1ull << (best / kWave);
    if (lane == 0) idx[(long)t * top + k] = best;
    if (lane == k % kWave) mine[k / kWave] = best_score;      // lane k keeps the k-th score until the sum is known
    picked += best_score;
  }
  const float inv = renorm ? scale / (picked + 1e-20f) : scale;
  for (int k = lane; k < top; k += kWave) wgt[(long)t * top + k] = mine[k / kWave] * inv;
}

// One workgroup.  tiles: [max_tiles][3] = (expert, first place in `sorted`, entries).
__global__ __launch_bounds__(1024) void moe_plan_kernel(const int* __restrict__ idx, int entries, int E, int max_tiles,
                                                        int tile_rows, int* __restrict__ sorted, int* __restrict__ tiles) {
  extern __shared__ int plan_lds[];
  int* counts = plan_lds;
  int* offs = plan_lds + E;
  int* cursor = plan_lds + 2 * E;
  for (int e = threadIdx.x; e < E; e += blockDim.x) counts[e] = cursor[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < entries; i += blockDim.x) {
    const int e = idx[i];
    if (e < E) atomicAdd(&counts[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int off = 0, nt = 0;
    for (int e = 0; e < E; ++e) {
      offs[e] = off;
      for (int s = 0; s < counts[e] && nt < max_tiles; s += tile_rows, ++nt) {
        tiles[3 * nt] = e;
        tiles[3 * nt + 1] = off + s;
        tiles[3 * nt + 2] = min(tile_rows, counts[e] - s);
      }
      off += counts[e];
    }
    for (; nt < max_tiles; ++nt) tiles[3 * nt] = tiles[3 * nt + 1] = tiles[3 * nt + 2] = 0;
  }
  __syncthreads();
  // Which place an entry gets among its expert's is left to the order of arrival: a row's
  // result does not depend on it.
  for (int i = threadIdx.x; i < entries; i += blockDim.x) {
    const int e = idx[i];
    if (e < E) sorted[offs[e] + atomicAdd(&cursor[e], 1)] = i;
  }
}

template <typename T> struct MoeOperand;
template <> struct MoeOperand<bf16_t> { typedef bf16x8 type; };
template <> struct MoeOperand<float> { typedef floatx4 type; };

__device__ __forceinline__ floatx16 moe_mfma(bf16x8 a, bf16x8 b, floatx16 acc) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
}
__device__ __forceinline__ floatx16 moe_mfma(floatx4 a, floatx4 b, floatx16 acc) {
#pragma unroll
  for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], b[e], acc, 0, 0, 0);
  return acc;
}

// Sixteen bytes of a row from element k0 on; zeros beyond the row's end.  `vec`: rows are
// multiples of 16 bytes long, so a chunk is whole or absent and 16-byte loads are aligned.
template <typename T>
__device__ __forceinline__ typename MoeOperand<T>::type moe_chunk(const T* __restrict__ row, int k0, int K, bool vec) {
  typedef typename MoeOperand<T>::type op_t;
  constexpr int EPC = 16 / sizeof(T);
  op_t v;
  if (vec) {
    if (k0 < K) return *reinterpret_cast<const op_t*>(row + k0);
#pragma unroll
    for (int j = 0; j < EPC; ++j) v[j] = (T)0.f;
    return v;
  }
#pragma unroll
  for (int j = 0; j < EPC; ++j) v[j] = k0 + j < K ? row[k0 + j] : (T)0.f;
  return v;
}

// MODE 0: X is the feed-forward's input [tokens, K]; W [E][2 M][K], an expert's gate rows, then its
//         up rows; out [entries, M] in T: the gated activation.
// MODE 1: X is [entries, K]; W [E][M][K]; out [entries, M] float32.
// Grid (tiles, column blocks).  A workgroup's four waves share a tile of 64 rows of X by 64
// columns (MODE 0: 64 gate rows and 64 up rows of W), 32 x 32 each, or of 128 rows by 128 columns
// (MODE 0: by 64, which is as many rows of W), 64 x 64 each: the larger tile asks the caches for
// fewer bytes a product, the smaller wastes less where an expert has few rows.  128 bytes of K of every row
// pass through LDS in two buffers: a thread asks memory for its 16-byte pieces of the next step,
// multiplies this step out of LDS, then puts the pieces down behind it.  Rows lie 144 bytes
// apart, so that the 16 lanes of a read meet 16 different groups of banks.  Which 16 bytes of
// K a lane multiplies in which of a step's four products is the same for both operands, which
// is all a product asks.
constexpr int kMoeRowBytes = 144;

template <typename T, int MODE, int MI, int NJ>    // a workgroup's tile: 64 MI rows by 64 NJ columns
__global__ __launch_bounds__(256) void moe_expert_kernel(const T* __restrict__ X, const T* __restrict__ W,
                                                         void* __restrict__ out_, const int* __restrict__ sorted,
                                                         const int* __restrict__ tiles, int top, int M, int K, int act,
                                                         float limit, float alpha) {
  typedef typename MoeOperand<T>::type op_t;
  constexpr int EPC = 16 / sizeof(T);
  constexpr int NB = MODE == 0 ? 2 : 1;           // blocks of rows of W: gate (and up)
  constexpr int AROWS = 64 * MI, BCOLS = 64 * NJ, BROWS = BCOLS * NB;
  constexpr int STAGE = (AROWS + BROWS) * kMoeRowBytes;
  constexpr int STEP = 8 * EPC;                   // elements of 128 bytes
  extern __shared__ __attribute__((aligned(16))) unsigned char moe_lds[];   // [2][STAGE]
  const int tile = blockIdx.x;
  const int count = tiles[3 * tile + 2];
  if (count == 0) return;
  const int expert = tiles[3 * tile], start = tiles[3 * tile + 1];
  const int c0 = blockIdx.y * BCOLS;
  if (c0 >= M) return;
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int wr = wave / 2, wc = wave % 2, r = lane % 32, half = lane / 32;   // a wave: 32 MI rows by 32 NJ columns
  const bool vec = K % EPC == 0;
  const T* wbase = W + (long)expert * NB * M * K;
  // what this thread brings in: piece `ch` of rows tid / 8 + 32 i of X and of W
  const int ch = tid % 8, row0 = tid / 8;
  const T* arow[AROWS / 32];
  const T* brow[BROWS / 32];
#pragma unroll
  for (int i = 0; i < AROWS / 32; ++i) {
    const int entry = sorted[start + min(row0 + 32 * i, count - 1)];
    arow[i] = X + (long)(MODE == 0 ? entry / top : entry) * K;
  }
#pragma unroll
  for (int i = 0; i < BROWS / 32; ++i) {
    const int row = row0 + 32 * i;                // the first BCOLS: gate (or the one product), then up
    brow[i] = wbase + ((long)(row / BCOLS) * M + min(c0 + row % BCOLS, M - 1)) * K;
  }
  op_t ra[AROWS / 32], rb[BROWS / 32];
  auto load = [&](int k) {
    const int k0 = k + ch * EPC;
#pragma unroll
    for (int i = 0; i < AROWS / 32; ++i) ra[i] = moe_chunk<T>(arow[i], k0, K, vec);
#pragma unroll
    for (int i = 0; i < BROWS / 32; ++i) rb[i] = moe_chunk<T>(brow[i], k0, K, vec);
  };
  auto put = [&](int buf) {
    unsigned char* base = moe_lds + buf * STAGE + ch * 16;
#pragma unroll
    for (int i = 0; i < AROWS / 32; ++i) *reinterpret_cast<op_t*>(base + (row0 + 32 * i) * kMoeRowBytes) = ra[i];
#pragma unroll
    for (int i = 0; i < BROWS / 32; ++i)
      *reinterpret_cast<op_t*>(base + (AROWS + row0 + 32 * i) * kMoeRowBytes) = rb[i];
  };
  floatx16 acc[MI][NJ][NB];
#pragma unroll
  for (int a = 0; a < MI; ++a)
#pragma unroll
    for (int b = 0; b < NJ; ++b)
#pragma unroll
      for (int g = 0; g < NB; ++g)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[a][b][g][e] = 0.f;
  load(0);
  put(0);
  __syncthreads();
  int buf = 0;
  for (int k = 0; k < K; k += STEP, buf ^= 1) {
    const bool more = k + STEP < K;
    if (more) load(k + STEP);
    const unsigned char* base = moe_lds + buf * STAGE;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int piece = (2 * i + half) * 16;
      op_t av[MI], bv[NJ][NB];
#pragma unroll
      for (int a = 0; a < MI; ++a)
        av[a] = *reinterpret_cast<const op_t*>(base + (wr * 32 * MI + 32 * a + r) * kMoeRowBytes + piece);
#pragma unroll
      for (int b = 0; b < NJ; ++b)
#pragma unroll
        for (int g = 0; g < NB; ++g)
          bv[b][g] = *reinterpret_cast<const op_t*>(
              base + (AROWS + g * BCOLS + wc * 32 * NJ + 32 * b + r) * kMoeRowBytes + piece);
#pragma unroll
      for (int a = 0; a < MI; ++a)
#pragma unroll
        for (int b = 0; b < NJ; ++b)
#pragma unroll
          for (int g = 0; g < NB; ++g) acc[a][b][g] = moe_mfma(av[a], bv[b][g], acc[a][b][g]);
    }
    if (more) put(buf ^ 1);
    __syncthreads();
  }
#pragma unroll
  for (int b = 0; b < NJ; ++b) {
    const int c = c0 + wc * 32 * NJ + 32 * b + r;
    if (c >= M) continue;
#pragma unroll
    for (int a = 0; a < MI; ++a)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = wr * 32 * MI + 32 * a + 8 * (e / 4) + 4 * half + e % 4;
        if (row >= count) continue;
        const long dst = (long)sorted[start + row] * M + c;
        if (MODE == 0)
          reinterpret_cast<T*>(out_)[dst] = from_f32<T>(gated(acc[a][b][0][e], acc[a][b][NB - 1][e], act, limit, alpha));
        else
          reinterpret_cast<float*>(out_)[dst] = acc[a][b][0][e];
      }
  }
}

template <typename T, int MODE, int MI, int NJ>
static int launch_moe_expert(const void* x, const void* w, void* out, const int* sorted, const int* tiles,
                             int max_tiles, int top, int m, int k, int act, float limit, float alpha,
                             hipStream_t stream) {
  const size_t lds = (size_t)2 * (64 * MI + 64 * NJ * (MODE == 0 ? 2 : 1)) * kMoeRowBytes;
  static int raised = 0;
  if (lds > 64 * 1024 && !raised) {
    hipError_t e = hipFuncSetAttribute((const void*)moe_expert_kernel<T, MODE, MI, NJ>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) KLLM_FAIL((int)e, "moe_expert: cannot raise the LDS limit: %s", hipGetErrorString(e));
    raised = 1;
  }
  const dim3 grid(max_tiles, ceil_div(m, 64 * NJ));
  hipLaunchKernelGGL((moe_expert_kernel<T, MODE, MI, NJ>), grid, dim3(256), lds, stream, (const T*)x, (const T*)w, out,
                     sorted, tiles, top, m, k, act, limit, alpha);
  return 0;
}

// The same products for few entries (decode batches), without tiles or a plan: a workgroup takes
// one entry and eight columns of its expert, two to a wave; a lane's share of K is every 64th
// piece of 16 bytes, all of a row's pieces asked for at once.  idx [entries]: the entry's expert
// (entries of experts from E on are skipped).
template <typename T>
__device__ __forceinline__ float moe_dot(typename MoeOperand<T>::type a, typename MoeOperand<T>::type b, float acc) {
  constexpr int EPC = 16 / sizeof(T);
#pragma unroll
  for (int j = 0; j < EPC; ++j) acc = fmaf(to_f32((T)a[j]), to_f32((T)b[j]), acc);
  return acc;
}

constexpr int kGemvCols = 2;       // columns a wave

template <typename T, int MODE>
__global__ __launch_bounds__(256) void moe_gemv_kernel(const T* __restrict__ X, const T* __restrict__ W,
                                                       void* __restrict__ out_, const int* __restrict__ idx, int E,
                                                       int top, int M, int K, int act, float limit, float alpha) {
  constexpr int EPC = 16 / sizeof(T);
  const int entry = blockIdx.x;
  const int expert = idx[entry];
  if (expert >= E) return;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int c0 = (blockIdx.y * 4 + wave) * kGemvCols;
  if (c0 >= M) return;
  const T* xrow = X + (long)(MODE == 0 ? entry / top : entry) * K;
  const T* wbase = W + (long)expert * (MODE == 0 ? 2 : 1) * M * K;
  const bool vec = K % EPC == 0;
  float g[kGemvCols], u[kGemvCols];
#pragma unroll
  for (int c = 0; c < kGemvCols; ++c) g[c] = u[c] = 0.f;
#pragma unroll 2
  for (int k = lane * EPC; k < K; k += kWave * EPC) {
    const auto a = moe_chunk<T>(xrow, k, K, vec);
#pragma unroll
    for (int c = 0; c < kGemvCols; ++c) {
      const int col = min(c0 + c, M - 1);
      g[c] = moe_dot<T>(a, moe_chunk<T>(wbase + (long)col * K, k, K, vec), g[c]);
      if (MODE == 0) u[c] = moe_dot<T>(a, moe_chunk<T>(wbase + (long)(M + col) * K, k, K, vec), u[c]);
    }
  }
#pragma unroll
  for (int c = 0; c < kGemvCols; ++c) {
    g[c] = wave_sum(g[c]);
    if (MODE == 0) u[c] = wave_sum(u[c]);
  }
  if (lane != 0) return;
#pragma unroll
  for (int c = 0; c < kGemvCols; ++c) {
    if (c0 + c >= M) continue;
    const long dst = (long)entry * M + c0 + c;
    if (MODE == 0)
      reinterpret_cast<T*>(out_)[dst] = from_f32<T>(gated(g[c], u[c], act, limit, alpha));
    else
      reinterpret_cast<float*>(out_)[dst] = g[c];
  }
}

template <typename T>
__global__ void moe_combine_kernel(const float* __restrict__ y, const T* __restrict__ xin, const int* __restrict__ idx,
                                   const float* __restrict__ wgt, const float* __restrict__ shared, int ns,
                                   long shared_stride, float* __restrict__ out, long count, int d, int top, int E,
                                   const float* __restrict__ shared_scale) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count) return;
  const long t = i / d;
  const int c = (int)(i % d);
  float v = 0.f;
  for (int s = 0; s < top; ++s) {
    const long entry = t * top + s;
    const float part = idx[entry] < E ? y[entry * d + c] : to_f32(xin[i]);
    v = fmaf(wgt[entry], part, v);
  }
  float sh = 0.f;
  for (int s = 0; s < ns; ++s) sh += shared[s * shared_stride + i];
  out[i] = shared_scale ? fmaf(shared_scale[t], sh, v) : v + sh;
}

}  // namespace kllm

using namespace kllm;

extern "C" int kllm_moe_tile_rows(void) { return kMoeTileRows; }

extern "C" int kllm_moe_route(const float* z, int nsplit, long split_stride, const float* correction, int n, int R,
                              int top, int* idx, float* wgt, int scoring, int groups, int keep, float scale, int renorm,
                              int cols, float* sgate, hipStream_t stream) {
  KLLM_REQUIRE(z && idx && wgt, "moe_route: null pointer");
  KLLM_REQUIRE((scoring == 0 || scoring == 1) && cols >= R + (sgate ? 1 : 0),
               "moe_route: scoring %d, or rows of %d sums for %d experts", scoring, cols, R);
  KLLM_REQUIRE(groups >= 1 && groups <= kWave && R % groups == 0 && keep >= 1 && keep <= groups &&
                   top <= R / groups * keep,
               "moe_route: %d groups (up to %d) of which %d are kept, for %d of %d experts", groups, kWave, keep, top, R);
  KLLM_REQUIRE(n > 0 && R > 0 && R <= kMaxRouted && top > 0 && top <= R && top <= kMaxTop && nsplit >= 1,
               "moe_route: bad sizes n=%d experts=%d (up to %d) top=%d (up to %d)", n, R, kMaxRouted, top, kMaxTop);
  hipLaunchKernelGGL(moe_route_kernel, dim3(ceil_div(n, 4)), dim3(256), 0, stream, z, nsplit, split_stride, correction,
                     n, R, top, idx, wgt, scoring, groups, keep, scale, renorm, cols, sgate);
  KLLM_CHECK_LAUNCH("moe_route");
  return 0;
}

extern "C" int kllm_moe_plan(const int* idx, int entries, int E, int max_tiles, int tile_rows, int* sorted,
                             int* tiles, hipStream_t stream) {
  KLLM_REQUIRE(idx && sorted && tiles, "moe_plan: null pointer");
  KLLM_REQUIRE(entries > 0 && E > 0 && E <= 4096, "moe_plan: bad sizes entries=%d experts=%d", entries, E);
  KLLM_REQUIRE(tile_rows == kMoeTileRows || tile_rows == 2 * kMoeTileRows, "moe_plan: tiles of %d rows are not built",
               tile_rows);
  KLLM_REQUIRE(max_tiles >= ceil_div(entries, tile_rows) + E, "moe_plan: %d tiles do not hold %d entries of %d experts",
               max_tiles, entries, E);
  hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(1024), (size_t)3 * E * sizeof(int), stream, idx, entries, E,
                     max_tiles, tile_rows, sorted, tiles);
  KLLM_CHECK_LAUNCH("moe_plan");
  return 0;
}

extern "C" int kllm_moe_expert(const void* x, const void* w, void* out, const int* sorted, const int* tiles,
                               int max_tiles, int tile_rows, int top, int m, int k, int mode, int act, float limit,
                               float alpha, int dtype, hipStream_t stream) {
  KLLM_REQUIRE(x && w && out && sorted && tiles, "moe_expert: null pointer");
  KLLM_REQUIRE(max_tiles > 0 && top > 0 && m > 0 && k > 0, "moe_expert: bad sizes tiles=%d top=%d m=%d k=%d", max_tiles,
               top, m, k);
  KLLM_REQUIRE(tile_rows == kMoeTileRows || tile_rows == 2 * kMoeTileRows, "moe_expert: tiles of %d rows are not built",
               tile_rows);
  KLLM_REQUIRE(mode == 0 || mode == 1, "moe_expert: mode %d", mode);
  KLLM_REQUIRE(mode == 1 || gated_known(act), "moe_expert: unknown activation %d", act);
  KLLM_REQUIRE(dtype == DT_F32 || dtype == DT_BF16, "moe_expert: unknown dtype %d", dtype);
  int rc;
#define KLLM_MOE(T, MODE)                                                                                        \
  rc = tile_rows == kMoeTileRows                                                                                 \
           ? launch_moe_expert<T, MODE, 1, 1>(x, w, out, sorted, tiles, max_tiles, top, m, k, act, limit, alpha, stream) \
           : launch_moe_expert<T, MODE, 2, MODE == 0 ? 1 : 2>(x, w, out, sorted, tiles, max_tiles, top, m, k, act, limit, \
                                                              alpha, stream)
  if (dtype == DT_F32) {
    if (mode == 0) KLLM_MOE(float, 0); else KLLM_MOE(float, 1);
  } else {
    if (mode == 0) KLLM_MOE(bf16_t, 0); else KLLM_MOE(bf16_t, 1);
  }
#undef KLLM_MOE
  if (rc) return rc;
  KLLM_CHECK_LAUNCH("moe_expert");
  return 0;
}

extern "C" int kllm_moe_expert_rows(const void* x, const void* w, void* out, const int* idx, int entries, int E,
                                    int top, int m, int k, int mode, int act, float limit, float alpha, int dtype,
                                    hipStream_t stream) {
  KLLM_REQUIRE(x && w && out && idx, "moe_expert_rows: null pointer");
  KLLM_REQUIRE(entries > 0 && entries <= 65535 && E > 0 && top > 0 && m > 0 && k > 0,
               "moe_expert_rows: bad sizes entries=%d E=%d top=%d m=%d k=%d", entries, E, top, m, k);
  KLLM_REQUIRE(mode == 0 || mode == 1, "moe_expert_rows: mode %d", mode);
  KLLM_REQUIRE(mode == 1 || gated_known(act), "moe_expert_rows: unknown activation %d", act);
  KLLM_REQUIRE(dtype == DT_F32 || dtype == DT_BF16, "moe_expert_rows: unknown dtype %d", dtype);
  const dim3 grid(entries, ceil_div(m, 4 * kGemvCols));
#define KLLM_MOE(T, MODE)                                                                                      \
  hipLaunchKernelGGL((moe_gemv_kernel<T, MODE>), grid, dim3(256), 0, stream, (const T*)x, (const T*)w, out, idx, E, \
                     top, m, k, act, limit, alpha)
  if (dtype == DT_F32) {
    if (mode == 0) KLLM_MOE(float, 0); else KLLM_MOE(float, 1);
  } else {
    if (mode == 0) KLLM_MOE(bf16_t, 0); else KLLM_MOE(bf16_t, 1);
  }
#undef KLLM_MOE
  KLLM_CHECK_LAUNCH("moe_expert_rows");
  return 0;
}

extern "C" int kllm_moe_combine(const float* y, const void* xin, const int* idx, const float* wgt, const float* shared,
                                int ns, long shared_stride, float* out, int n, int d, int top, int E, int dtype,
                                const float* shared_scale, hipStream_t stream) {
  KLLM_REQUIRE(y && xin && idx && wgt && out, "moe_combine: null pointer");
  KLLM_REQUIRE(n > 0 && d > 0 && top > 0 && E >= 0 && ns >= 0, "moe_combine: bad sizes n=%d d=%d top=%d", n, d, top);
  KLLM_REQUIRE(shared || ns == 0, "moe_combine: slices of a shared expert without its sums");
  KLLM_REQUIRE(dtype == DT_F32 || dtype == DT_BF16, "moe_combine: unknown dtype %d", dtype);
  const long count = (long)n * d;
  const dim3 grid(ceil_div(count, 256));
  if (dtype == DT_F32)
    hipLaunchKernelGGL(moe_combine_kernel<float>, grid, dim3(256), 0, stream, y, (const float*)xin, idx, wgt, shared, ns,
                       shared_stride, out, count, d, top, E, shared_scale);
  else
    hipLaunchKernelGGL(moe_combine_kernel<bf16_t>, grid, dim3(256), 0, stream, y, (const bf16_t*)xin, idx, wgt, shared,
                       ns, shared_stride, out, count, d, top, E, shared_scale);
  KLLM_CHECK_LAUNCH("moe_combine");
  return 0;
}
