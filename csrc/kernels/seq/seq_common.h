// Shared device helpers of the stateful-model kernels (csrc/kernels/seq): element types and
// conversions.  Element type codes of the C API: 0 = fp32, 1 = bf16.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint16_t bf16_t;   // raw bfloat16 bits

__device__ __forceinline__ float bf16_to_f(bf16_t v) { return __uint_as_float(((uint32_t)v) << 16); }
__device__ __forceinline__ bf16_t f_to_bf16(float f) {          // round to nearest even
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x40);   // NaN stays NaN
  u += 0x7fffu + ((u >> 16) & 1u);
  return (bf16_t)(u >> 16);
}
__device__ __forceinline__ float ldf(const float* p, size_t i) { return p[i]; }
__device__ __forceinline__ float ldf(const bf16_t* p, size_t i) { return bf16_to_f(p[i]); }
__device__ __forceinline__ void stf(float* p, size_t i, float v) { p[i] = v; }
__device__ __forceinline__ void stf(bf16_t* p, size_t i, float v) { p[i] = f_to_bf16(v); }

__device__ __forceinline__ float wave_max(float v) {
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
// sum over the 256 threads of a block (red: 4 floats of LDS); every thread gets the result
__device__ __forceinline__ float block_sum_256(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return red[0] + red[1] + red[2] + red[3];
}
__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }
__device__ __forceinline__ float sigmoid_f(float z) { return 1.f / (1.f + expf(-z)); }
__device__ __forceinline__ float silu_f(float z) { return z / (1.f + expf(-z)); }
// gelu, tanh form: 0.5 z (1 + tanh(u)) with u = sqrt(2/pi) (z + 0.044715 z^3), written as z sigmoid(2u):
// one exponential, and no cancellation in the negative tail
__device__ __forceinline__ float gelu_tanh_f(float z) {
  return z / (1.f + expf(-1.5957691216057308f * (z + 0.044715f * z * z * z)));
}

// attn_paged.hip: out[t, h] from nsplit partial (maximum, sum, weighted values) records per (row, head)
typedef void* fls_stream_t;
// has_sink: the softmax's silent entry of score `sink` joins the total here; head_gate (nullable) [T, H]: a sigmoid gate per (row, head)
int seq_attn_merge(const float* part, void* out, int tc, int ldo, int T, int H, int dv, int nsplit, int gated, float out_scale,
                   int has_sink, float sink, const float* head_gate, int ldhg, fls_stream_t s);

#define SEQ_LAUNCH_CHECK() do { hipError_t e_ = hipGetLastError(); if (e_ != hipSuccess) return (int)e_; } while (0)
