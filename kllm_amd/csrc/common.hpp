// Shared declarations of the gfx950 kernels: storage types, conversions,
// wave reductions, error reporting and launch checks.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

namespace kllm {

constexpr int kWave = 64;  // CDNA wavefront

// Storage types of weights, activations and cache. DT_F32 / DT_BF16 are the
// values of the `dtype` argument of every entry point.
enum : int { DT_F32 = 0, DT_BF16 = 1 };
typedef __bf16 bf16_t;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return (float)v; }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
// float -> bfloat16 rounds to nearest even (the hardware conversion of gfx950).
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return (bf16_t)v; }

// The gate's activation of a gated feed-forward, the value of the `act` argument of the
// entry points that apply one.  Another activation is another value here and another case
// in gate_act; every kernel with a gate in its epilogue calls this one function.
enum : int { ACT_SILU = 0, ACT_GELU_TANH = 1, ACT_COUNT = 2 };

__device__ __forceinline__ float gate_act(float g, int act) {
  if (act == ACT_GELU_TANH) {   // 0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3)))
    const float u = 0.7978845608028654f * (g + 0.044715f * g * g * g);
    return 0.5f * g * (1.f + tanhf(u));
  }
  return g / (1.f + expf(-g));  // SiLU (reference: backend/model.cu:477-483)
}

// Activations without a gate (kllm_unary_act): the gates' two, and xIELU, whose two constants
// are learned: for z > 0, a_pos z^2 + z/2; otherwise (1/2 + a_neg) (exp(z) - 1 - z) + z/2.
// The square of the rectifier: max(z, 0)^2.  The identity (sums that only change their type) and
// the logistic function.
enum : int { ACT_XIELU = 2, ACT_TANH = 3, ACT_RELU_SQ = 4, ACT_IDENTITY = 5, ACT_SIGMOID = 6, UNARY_ACT_COUNT = 7 };

__device__ __forceinline__ float softplus_f32(float v) { return v > 20.f ? v : log1pf(expf(v)); }

__device__ __forceinline__ float unary_act(float z, int act, float a_pos, float a_neg) {
  if (act == ACT_XIELU)
    return z > 0.f ? fmaf(a_pos * z, z, 0.5f * z) : fmaf(0.5f + a_neg, expm1f(z) - z, 0.5f * z);
  if (act == ACT_TANH) return tanhf(z);
  if (act == ACT_IDENTITY) return z;
  if (act == ACT_SIGMOID) return 1.f / (1.f + expf(-z));
  if (act == ACT_RELU_SQ) {
    const float p = fmaxf(z, 0.f);
    return p * p;
  }
  return gate_act(z, act);
}

// The first key that the query at position `pos` reads: with a window the last `window`
// positions, with a chunked mask nothing before the start of the query's own chunk of
// `chunk` positions (chunks are counted from position 0); 0 switches either off.  Both
// bounds grow with the position, which the kernels that take blocks of queries rely on.
__host__ __device__ __forceinline__ int first_key(int pos, int window, int chunk) {
  int start = (window > 0 && pos + 1 > window) ? pos + 1 - window : 0;
  if (chunk > 0) {
    const int c = pos - pos % chunk;
    start = c > start ? c : start;
  }
  return start;
}

__device__ __forceinline__ float sigmoid_f32(float v) { return 1.f / (1.f + expf(-v)); }

// A gate and the sum it gates, for kernels that take both: act(g) * u for the gates' activations,
// or the clamped gate: with g' = min(g, limit) and u' = clamp(u, -limit, limit),
// g' sigmoid(alpha g') (u' + 1).
enum : int { GATE_CLAMPED_SWISH = 4, GATED_COUNT = 5 };

__host__ __device__ __forceinline__ bool gated_known(int act) { return (act >= 0 && act < ACT_COUNT) || act == GATE_CLAMPED_SWISH; }

__device__ __forceinline__ float gated(float g, float u, int act, float limit, float alpha) {
  if (act == GATE_CLAMPED_SWISH) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return g * sigmoid_f32(alpha * g) * (u + 1.f);
  }
  return gate_act(g, act) * u;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}

// Sum over a workgroup of up to 1024 threads. `red` is LDS of at least 16
// floats. Every thread gets the result; the order of additions is fixed.
__device__ __forceinline__ float block_sum(float v, float* red) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int nwaves = (blockDim.x + kWave - 1) / kWave;
  v = wave_sum(v);
  __syncthreads();  // red may still be read from an earlier call
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < nwaves; ++w) total += red[w];
  return total;
}

__device__ __forceinline__ float block_max(float v, float* red) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int nwaves = (blockDim.x + kWave - 1) / kWave;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float total = red[0];
  for (int w = 1; w < nwaves; ++w) total = fmaxf(total, red[w]);
  return total;
}

// ---- errors ---------------------------------------------------------------
// Return convention of every entry point: 0 ok; a positive value is a HIP
// error code; negative values are ERR_ARG (a size or pointer the kernel does
// not take) and ERR_STATE.  The text of the calling thread's last error is
// read with kllm_last_error.
enum : int { ERR_ARG = -2, ERR_STATE = -1 };

void set_error(const char* fmt, ...);

#define KLLM_FAIL(code, ...)            \
  do {                                  \
    ::kllm::set_error(__VA_ARGS__);     \
    return (code);                      \
  } while (0)

#define KLLM_REQUIRE(cond, ...)                   \
  do {                                            \
    if (!(cond)) KLLM_FAIL(::kllm::ERR_ARG, __VA_ARGS__); \
  } while (0)

#define KLLM_CHECK_LAUNCH(name)                                                   \
  do {                                                                            \
    hipError_t e_ = hipGetLastError();                                            \
    if (e_ != hipSuccess)                                                         \
      KLLM_FAIL((int)e_, "%s: launch failed: %s", name, hipGetErrorString(e_));   \
  } while (0)

// Compute units of the current device (cached); 256 if it cannot be asked.
int device_cus();
// XCDs of the current device (cached); 8 if it cannot be asked.
int device_xcds();

inline int ceil_div(long a, long b) { return (int)((a + b - 1) / b); }

// Sum over the PARTS neighbouring lanes that share a column (PARTS a power of two up to 64), every
// lane getting the sum: within a row of 16 lanes by data-parallel moves (neighbour, other pair,
// mirrored half row, mirrored row), which cost an instruction each; across the two rows of a
// group of 32 by a lane exchange.
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
  const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true);   // (every lane has a source: the move folds into the add)
  return v + __builtin_bit_cast(float, moved);
}

template <int PARTS>
__device__ __forceinline__ float parts_sum(float v) {
  if (PARTS >= 2) v = dpp_add<0xB1>(v);     // quad_perm [1,0,3,2]
  if (PARTS >= 4) v = dpp_add<0x4E>(v);     // quad_perm [2,3,0,1]
  if (PARTS >= 8) v = dpp_add<0x141>(v);    // row_half_mirror
  if (PARTS >= 16) v = dpp_add<0x140>(v);   // row_mirror
  if (PARTS >= 32) v += __shfl_xor(v, 16, kWave);
  if (PARTS >= 64) v += __shfl_xor(v, 32, kWave);
  return v;
}

}  // namespace kllm
