// Row-wise kernels of the stateful models: group RMS norm (also as the residual update), embedding
// gather into the fp32 residual stream, activations between GEMMs, logit cap, K/V store with the key
// norm, and the routing of a mixture of experts.  All statistics and sums are fp32.
#include "seq_common.h"
#include "fls_seq.h"

// ------------------------------------------------------------------------- group RMS norm
// one block per (row, group): sum of squares of D / groups columns, then the scaled row part
template <typename TO, int ADD>
__global__ __launch_bounds__(256) void group_rmsnorm_kernel(const float* __restrict__ x, int ldx, const int* __restrict__ idx,
                                                            const float* __restrict__ w, TO* __restrict__ y, int ldy,
                                                            int D, int groups, float eps, float woff) {
  __shared__ float red[4];
  const int r = blockIdx.x, g = blockIdx.y;
  const int n = D / groups;
  const float* xr = x + (size_t)(idx != nullptr ? idx[r] : r) * ldx + (size_t)g * n;
  float ss = 0.f;
  for (int c = threadIdx.x; c < n; c += 256) { const float v = xr[c]; ss += v * v; }
  ss = block_sum_256(ss, red);
  const float rs = 1.f / sqrtf(ss / (float)n + eps);
  const float* wg = w + (size_t)g * n;
  TO* yr = y + (size_t)r * ldy + (size_t)g * n;
  for (int c = threadIdx.x; c < n; c += 256) {
    const float v = xr[c] * rs * (wg[c] + woff);
    if constexpr (ADD) yr[c] += v; else stf(yr, c, v);
  }
}

extern "C" int fls_seq_group_rmsnorm(const float* x, int ldx, const int* idx, const float* w, void* y, int ty, int ldy,
                                     int rows, int D, int groups, float eps, int add, float woff, fls_stream_t s) {
  if (rows <= 0) return 0;
  if (groups < 1 || D % groups) return -1;
  dim3 grid(rows, groups);
  hipStream_t st = (hipStream_t)s;
  if (add) hipLaunchKernelGGL((group_rmsnorm_kernel<float, 1>), grid, dim3(256), 0, st, x, ldx, idx, w, (float*)y, ldy, D, groups, eps, woff);
  else if (ty == 1) hipLaunchKernelGGL((group_rmsnorm_kernel<bf16_t, 0>), grid, dim3(256), 0, st, x, ldx, idx, w, (bf16_t*)y, ldy, D, groups, eps, woff);
  else hipLaunchKernelGGL((group_rmsnorm_kernel<float, 0>), grid, dim3(256), 0, st, x, ldx, idx, w, (float*)y, ldy, D, groups, eps, woff);
  SEQ_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------------- Dynamic Tanh norm
// y[r, c] = tanh(alpha x[row, c]) w[c] + b[c]: no statistic of the row, so the work is cut over
// (row, 1024-column piece) blocks of four columns a thread.  wb = [w; b], alpha one number on the device.
template <typename TO>
__global__ __launch_bounds__(256) void dyt_norm_kernel(const float* __restrict__ x, int ldx, const int* __restrict__ idx,
                                                       const float* __restrict__ wb, const float* __restrict__ alpha,
                                                       TO* __restrict__ y, int ldy, int D, int vec) {
  const int r = blockIdx.x;
  const float a = alpha[0];
  const float* xr = x + (size_t)(idx != nullptr ? idx[r] : r) * ldx;
  const float* w = wb;
  const float* b = wb + D;
  TO* yr = y + (size_t)r * ldy;
  const int c0 = (blockIdx.y * 256 + threadIdx.x) * 4;
  if (c0 >= D) return;
  if (vec) {
    const float4 v = *reinterpret_cast<const float4*>(xr + c0);
    const float4 wv = *reinterpret_cast<const float4*>(w + c0), bv = *reinterpret_cast<const float4*>(b + c0);
    const float o0 = tanhf(a * v.x) * wv.x + bv.x, o1 = tanhf(a * v.y) * wv.y + bv.y;
    const float o2 = tanhf(a * v.z) * wv.z + bv.z, o3 = tanhf(a * v.w) * wv.w + bv.w;
    if constexpr (sizeof(TO) == 2) {
      bf16_t e[4] = {f_to_bf16(o0), f_to_bf16(o1), f_to_bf16(o2), f_to_bf16(o3)};
      *reinterpret_cast<uint2*>(yr + c0) = *reinterpret_cast<const uint2*>(e);
    } else {
      *reinterpret_cast<float4*>(yr + c0) = make_float4(o0, o1, o2, o3);
    }
  } else {
    for (int c = c0; c < min(D, c0 + 4); ++c) stf(yr, c, tanhf(a * xr[c]) * w[c] + b[c]);
  }
}

extern "C" int fls_seq_dyt_norm(const float* x, int ldx, const int* idx, const float* wb, const float* alpha, void* y, int ty,
                                int ldy, int rows, int D, fls_stream_t s) {
  if (rows <= 0) return 0;
  if (D < 1) return -1;
  const int vec = D % 4 == 0 && ldx % 4 == 0 && ldy % 4 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)wb % 16 == 0 &&
                  (uintptr_t)y % 16 == 0;
  dim3 grid(rows, (D + 1023) / 1024);
  hipStream_t st = (hipStream_t)s;
  if (ty == 1) hipLaunchKernelGGL((dyt_norm_kernel<bf16_t>), grid, dim3(256), 0, st, x, ldx, idx, wb, alpha, (bf16_t*)y, ldy, D, vec);
  else hipLaunchKernelGGL((dyt_norm_kernel<float>), grid, dim3(256), 0, st, x, ldx, idx, wb, alpha, (float*)y, ldy, D, vec);
  SEQ_LAUNCH_CHECK();
  return 0;
}

// x[r, c] += mult * y[r, c]: a sublayer's output joins the residual stream scaled
__global__ __launch_bounds__(256) void add_scaled_kernel(float* __restrict__ x, int ldx, const float* __restrict__ y, int ldy, int D,
                                                         float mult, int vec) {
  float* xr = x + (size_t)blockIdx.x * ldx;
  const float* yr = y + (size_t)blockIdx.x * ldy;
  const int c0 = (blockIdx.y * 256 + threadIdx.x) * 4;
  if (c0 >= D) return;
  if (vec) {
    float4 a = *reinterpret_cast<const float4*>(xr + c0);
    const float4 b = *reinterpret_cast<const float4*>(yr + c0);
    a.x += mult * b.x; a.y += mult * b.y; a.z += mult * b.z; a.w += mult * b.w;
    *reinterpret_cast<float4*>(xr + c0) = a;
  } else {
    for (int c = c0; c < min(D, c0 + 4); ++c) xr[c] += mult * yr[c];
  }
}

extern "C" int fls_seq_add_scaled(float* x, int ldx, const float* y, int ldy, int rows, int D, float mult, fls_stream_t s) {
  if (rows <= 0) return 0;
  const int vec = D % 4 == 0 && ldx % 4 == 0 && ldy % 4 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)y % 16 == 0;
  hipLaunchKernelGGL(add_scaled_kernel, dim3(rows, (D + 1023) / 1024), dim3(256), 0, (hipStream_t)s, x, ldx, y, ldy, D, mult, vec);
  SEQ_LAUNCH_CHECK();
  return 0;
}

// x[r, c] += mult * y[r, c] and h[r, c] = tanh(alpha x[r, c]) w[c] + b[c] of the new x: the residual update and the
// next sublayer's Dynamic Tanh norm in one pass over the stream
template <typename TO>
__global__ __launch_bounds__(256) void add_scaled_dyt_kernel(float* __restrict__ x, int ldx, const float* __restrict__ y, int ldy,
                                                             float mult, const float* __restrict__ wb,
                                                             const float* __restrict__ alpha, TO* __restrict__ h, int ldh,
                                                             int D, int vec) {
  const float a = alpha[0];
  float* xr = x + (size_t)blockIdx.x * ldx;
  const float* yr = y + (size_t)blockIdx.x * ldy;
  TO* hr = h + (size_t)blockIdx.x * ldh;
  const float* w = wb;
  const float* b = wb + D;
  const int c0 = (blockIdx.y * 256 + threadIdx.x) * 4;
  if (c0 >= D) return;
  if (vec) {
    float4 v = *reinterpret_cast<const float4*>(xr + c0);
    const float4 u = *reinterpret_cast<const float4*>(yr + c0);
    v.x += mult * u.x; v.y += mult * u.y; v.z += mult * u.z; v.w += mult * u.w;
    *reinterpret_cast<float4*>(xr + c0) = v;
    const float4 wv = *reinterpret_cast<const float4*>(w + c0), bv = *reinterpret_cast<const float4*>(b + c0);
    const float o0 = tanhf(a * v.x) * wv.x + bv.x, o1 = tanhf(a * v.y) * wv.y + bv.y;
    const float o2 = tanhf(a * v.z) * wv.z + bv.z, o3 = tanhf(a * v.w) * wv.w + bv.w;
    if constexpr (sizeof(TO) == 2) {
      bf16_t e[4] = {f_to_bf16(o0), f_to_bf16(o1), f_to_bf16(o2), f_to_bf16(o3)};
      *reinterpret_cast<uint2*>(hr + c0) = *reinterpret_cast<const uint2*>(e);
    } else {
      *reinterpret_cast<float4*>(hr + c0) = make_float4(o0, o1, o2, o3);
    }
  } else {
    for (int c = c0; c < min(D, c0 + 4); ++c) {
      const float v = xr[c] + mult * yr[c];
      xr[c] = v;
      stf(hr, c, tanhf(a * v) * w[c] + b[c]);
    }
  }
}

extern "C" int fls_seq_add_scaled_dyt(float* x, int ldx, const float* y, int ldy, float mult, const float* wb, const float* alpha,
                                      void* h, int th, int ldh, int rows, int D, fls_stream_t s) {
  if (rows <= 0) return 0;
  const int vec = D % 4 == 0 && ldx % 4 == 0 && ldy % 4 == 0 && ldh % 4 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)y % 16 == 0 &&
                  (uintptr_t)wb % 16 == 0 && (uintptr_t)h % 16 == 0;
  dim3 grid(rows, (D + 1023) / 1024);
  hipStream_t st = (hipStream_t)s;
  if (th == 1) hipLaunchKernelGGL((add_scaled_dyt_kernel<bf16_t>), grid, dim3(256), 0, st, x, ldx, y, ldy, mult, wb, alpha, (bf16_t*)h, ldh, D, vec);
  else hipLaunchKernelGGL((add_scaled_dyt_kernel<float>), grid, dim3(256), 0, st, x, ldx, y, ldy, mult, wb, alpha, (float*)h, ldh, D, vec);
  SEQ_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------------------- embedding
template <typename T>
__global__ void embed_kernel(const int* __restrict__ ids, const T* __restrict__ table, float* __restrict__ out, int D, int V, float scale) {
  const int t = blockIdx.x;
  int id = ids[t];
  id = id < 0 ? 0 : (id >= V ? V - 1 : id);
  const T* row = table + (size_t)id * D;
  for (int c = threadIdx.x; c < D; c += blockDim.x) out[(size_t)t * D + c] = ldf(row, c) * scale;
}

extern "C" int fls_seq_embed(const int* ids, const void* table, int tt, float* out, int T, int D, int V, float scale, fls_stream_t s) {
  if (T <= 0) return 0;
  if (tt == 1) hipLaunchKernelGGL((embed_kernel<bf16_t>), dim3(T), dim3(256), 0, (hipStream_t)s, ids, (const bf16_t*)table, out, D, V, scale);
  else hipLaunchKernelGGL((embed_kernel<float>), dim3(T), dim3(256), 0, (hipStream_t)s, ids, (const float*)table, out, D, V, scale);
  SEQ_LAUNCH_CHECK();
  return 0;
}

template <typename T>
__global__ void gather_rows_kernel(const T* __restrict__ x, int ldx, const int* __restrict__ idx, T* __restrict__ y, int ldy, int D) {
  const T* xr = x + (size_t)idx[blockIdx.x] * ldx;
  T* yr = y + (size_t)blockIdx.x * ldy;
  for (int c = threadIdx.x; c < D; c += blockDim.x) yr[c] = xr[c];
}

extern "C" int fls_seq_gather_rows(const void* x, int tx, int ldx, const int* idx, void* y, int ldy, int rows, int D,
                                   fls_stream_t s) {
  if (rows <= 0) return 0;
  if (tx == 1) hipLaunchKernelGGL((gather_rows_kernel<bf16_t>), dim3(rows), dim3(256), 0, (hipStream_t)s, (const bf16_t*)x, ldx, idx, (bf16_t*)y, ldy, D);
  else hipLaunchKernelGGL((gather_rows_kernel<float>), dim3(rows), dim3(256), 0, (hipStream_t)s, (const float*)x, ldx, idx, (float*)y, ldy, D);
  SEQ_LAUNCH_CHECK();
  return 0;
}

// --------------------------------------------------------------------- activations between GEMMs
template <typename TO>
__global__ void xielu_kernel(const float* __restrict__ z, int ldz, const float* __restrict__ act, TO* __restrict__ y, int ldy, int cols) {
  const float ap = softplus_f(act[0]), an = 0.5f + softplus_f(act[1]);
  const float* zr = z + (size_t)blockIdx.x * ldz;
  TO* yr = y + (size_t)blockIdx.x * ldy;
  for (int c = threadIdx.x; c < cols; c += blockDim.x) {
    const float v = zr[c];
    stf(yr, c, v > 0.f ? ap * v * v + 0.5f * v : an * (expm1f(v) - v) + 0.5f * v);
  }
}

extern "C" int fls_seq_xielu(const float* z, int ldz, const float* act, void* y, int ty, int ldy, int rows, int cols, fls_stream_t s) {
  if (rows <= 0) return 0;
  if (ty == 1) hipLaunchKernelGGL((xielu_kernel<bf16_t>), dim3(rows), dim3(256), 0, (hipStream_t)s, z, ldz, act, (bf16_t*)y, ldy, cols);
  else hipLaunchKernelGGL((xielu_kernel<float>), dim3(rows), dim3(256), 0, (hipStream_t)s, z, ldz, act, (float*)y, ldy, cols);
  SEQ_LAUNCH_CHECK();
  return 0;
}

// y = act(gate) * up for rows [gate | up]; act: 0 = silu, 1 = gelu (tanh form)
template <typename TO, int ACT>
__global__ void gate_mul_kernel(const float* __restrict__ gu, int ldg, TO* __restrict__ y, int ldy, int cols) {
  const float* gr = gu + (size_t)blockIdx.x * ldg;
  TO* yr = y + (size_t)blockIdx.x * ldy;
  for (int c = threadIdx.x; c < cols; c += blockDim.x)
    stf(yr, c, (ACT == 1 ? gelu_tanh_f(gr[c]) : silu_f(gr[c])) * gr[cols + c]);
}

extern "C" int fls_seq_gate_mul(const float* gu, int ldg, void* y, int ty, int ldy, int rows, int cols, int act, fls_stream_t s) {
  if (rows <= 0) return 0;
  if (act < 0 || act > 1) return -1;
  hipStream_t st = (hipStream_t)s;
  if (ty == 1 && act == 0) hipLaunchKernelGGL((gate_mul_kernel<bf16_t, 0>), dim3(rows), dim3(256), 0, st, gu, ldg, (bf16_t*)y, ldy, cols);
  else if (ty == 1) hipLaunchKernelGGL((gate_mul_kernel<bf16_t, 1>), dim3(rows), dim3(256), 0, st, gu, ldg, (bf16_t*)y, ldy, cols);
  else if (act == 0) hipLaunchKernelGGL((gate_mul_kernel<float, 0>), dim3(rows), dim3(256), 0, st, gu, ldg, (float*)y, ldy, cols);
  else hipLaunchKernelGGL((gate_mul_kernel<float, 1>), dim3(rows), dim3(256), 0, st, gu, ldg, (float*)y, ldy, cols);
  SEQ_LAUNCH_CHECK();
  return 0;
}

// y = f(z) elementwise; kind: 0 = tanh, 1 = gelu in its exact form 0.5 z (1 + erf(z / sqrt 2))
template <typename TO>
__global__ void unary_kernel(const float* __restrict__ z, int ldz, TO* __restrict__ y, int ldy, int cols, int kind) {
  const float* zr = z + (size_t)blockIdx.x * ldz;
  TO* yr = y + (size_t)blockIdx.x * ldy;
  if (kind == 1) {
    for (int c = threadIdx.x; c < cols; c += blockDim.x) { const float v = zr[c]; stf(yr, c, 0.5f * v * (1.f + erff(v * 0.70710678118654752f))); }
    return;
  }
  for (int c = threadIdx.x; c < cols; c += blockDim.x) stf(yr, c, tanhf(zr[c]));
}

extern "C" int fls_seq_unary(const float* z, int ldz, void* y, int ty, int ldy, int rows, int cols, int kind, fls_stream_t s) {
  if (rows <= 0) return 0;
  if (kind != 0 && kind != 1) return -1;
  if (ty == 1) hipLaunchKernelGGL((unary_kernel<bf16_t>), dim3(rows), dim3(256), 0, (hipStream_t)s, z, ldz, (bf16_t*)y, ldy, cols, kind);
  else hipLaunchKernelGGL((unary_kernel<float>), dim3(rows), dim3(256), 0, (hipStream_t)s, z, ldz, (float*)y, ldy, cols, kind);
  SEQ_LAUNCH_CHECK();
  return 0;
}

__global__ void softcap_kernel(float* __restrict__ z, int ldz, int cols, float cap) {
  float* zr = z + (size_t)blockIdx.x * ldz;
  for (int c = threadIdx.x; c < cols; c += blockDim.x) zr[c] = cap * tanhf(zr[c] / cap);
}

extern "C" int fls_seq_softcap(float* z, int ldz, int rows, int cols, float cap, fls_stream_t s) {
  if (rows <= 0) return 0;
  hipLaunchKernelGGL(softcap_kernel, dim3(rows), dim3(256), 0, (hipStream_t)s, z, ldz, cols, cap);
  SEQ_LAUNCH_CHECK();
  return 0;
}

// first index of the row maximum
__global__ __launch_bounds__(256) void argmax_kernel(const float* __restrict__ z, int ldz, int cols, int* __restrict__ out) {
  __shared__ float bv[256];
  __shared__ int bi[256];
  const float* zr = z + (size_t)blockIdx.x * ldz;
  float best = -INFINITY;
  int at = 0x7fffffff;
  for (int c = threadIdx.x; c < cols; c += 256) {
    const float v = zr[c];
    if (v > best || (v == best && c < at)) { best = v; at = c; }
  }
  bv[threadIdx.x] = best;
  bi[threadIdx.x] = at;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) {
    if ((int)threadIdx.x < o) {
      const float v = bv[threadIdx.x + o];
      const int i = bi[threadIdx.x + o];
      if (v > bv[threadIdx.x] || (v == bv[threadIdx.x] && i < bi[threadIdx.x])) { bv[threadIdx.x] = v; bi[threadIdx.x] = i; }
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) out[blockIdx.x] = bi[0] == 0x7fffffff ? 0 : bi[0];
}

extern "C" int fls_seq_argmax(const float* z, int ldz, int rows, int cols, int* out, fls_stream_t s) {
  if (rows <= 0) return 0;
  hipLaunchKernelGGL(argmax_kernel, dim3(rows), dim3(256), 0, (hipStream_t)s, z, ldz, cols, out);
  SEQ_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------- K/V store with the key norm
template <typename TC>
__global__ __launch_bounds__(256) void kv_store_kernel(const float* __restrict__ k, int ldk, const float* __restrict__ kn, float eps,
                                                       const float* __restrict__ v, int ldv, TC* __restrict__ kc, TC* __restrict__ vc,
                                                       const int* __restrict__ kv_slot, int kcols, int vcols) {
  __shared__ float red[4];
  const int r = blockIdx.x;
  const float* kr = k + (size_t)r * ldk;
  float ss = 0.f;
  for (int c = threadIdx.x; c < kcols; c += 256) { const float x = kr[c]; ss += x * x; }
  ss = block_sum_256(ss, red);
  const float rs = 1.f / sqrtf(ss / (float)kcols + eps);
  const size_t dst = (size_t)kv_slot[r];
  for (int c = threadIdx.x; c < kcols; c += 256) stf(kc + dst * kcols, c, kr[c] * rs * kn[c]);
  const float* vr = v + (size_t)r * ldv;
  for (int c = threadIdx.x; c < vcols; c += 256) stf(vc + dst * vcols, c, vr[c]);
}

extern "C" int fls_seq_kv_store(const float* k, int ldk, const float* kn, float eps, const float* v, int ldv, void* kc, void* vc,
                                int tc, const int* kv_slot, int rows, int kcols, int vcols, fls_stream_t s) {
  if (rows <= 0) return 0;
  if (tc == 1) hipLaunchKernelGGL((kv_store_kernel<bf16_t>), dim3(rows), dim3(256), 0, (hipStream_t)s, k, ldk, kn, eps, v, ldv, (bf16_t*)kc, (bf16_t*)vc, kv_slot, kcols, vcols);
  else hipLaunchKernelGGL((kv_store_kernel<float>), dim3(rows), dim3(256), 0, (hipStream_t)s, k, ldk, kn, eps, v, ldv, (float*)kc, (float*)vc, kv_slot, kcols, vcols);
  SEQ_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------- per-head norm, rotation and placement
// One wave per (row, head): the head's n entries x[t, x_col + h x_hs ...] are RMS-normed over n (when w
// is given: times w[n], one weight for all heads), their first `rot` entries rotated in pairs
// (2i, 2i + 1) by the angle pos[t] * freqs[i] (fp32 angle, full-range sin / cos), and written to
// out[row, out_col + h out_hs ...] with row = row_map ? row_map[t] : t -- a matrix of rows or a page
// pool.  raw (optional, laid out like out) receives the entries as they came.  n <= 512.
#define HNR_MAX_E 8
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void head_norm_rope_kernel(const TI* x, int ldx, int x_col, int x_hs, int heads, int n,
                                                             const float* __restrict__ w, float eps,
                                                             const float* __restrict__ freqs, int rot,
                                                             const int* __restrict__ tok_pos, const int* __restrict__ row_map,
                                                             TO* out, int ldo, int out_col, int out_hs, TO* raw, int ldr,
                                                             int items, int unit_after, int half, float amp) {
  const int lane = threadIdx.x & 63;
  const int item = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= items) return;
  const int t = item / heads, h = item % heads;
  const TI* xr = x + (size_t)t * ldx + x_col + (size_t)h * x_hs;
  float v[HNR_MAX_E];
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < HNR_MAX_E; ++e) {
    const int c = lane + 64 * e;
    v[e] = c < n ? ldf(xr, c) : 0.f;
    ss += v[e] * v[e];
  }
  const size_t row = row_map != nullptr ? (size_t)row_map[t] : (size_t)t;
  if (raw != nullptr) {
    TO* rr = raw + row * ldr + out_col + (size_t)h * out_hs;
#pragma unroll
    for (int e = 0; e < HNR_MAX_E; ++e) { const int c = lane + 64 * e; if (c < n) stf(rr, c, v[e]); }
  }
  float rs_w = 1.f;
  if (w != nullptr) {
    const float rs = 1.f / sqrtf(wave_sum(ss) / (float)n + eps);
    rs_w = rs;
#pragma unroll
    for (int e = 0; e < HNR_MAX_E; ++e) { const int c = lane + 64 * e; if (c < n) v[e] *= rs * w[c]; }
  }
  const float pos = rot > 0 ? (float)tok_pos[t] : 0.f;
  TO* orow = out + row * ldo + out_col + (size_t)h * out_hs;
  // the pair's other entry: in the neighbouring lane for pairs (2i, 2i + 1); for pairs (i, i + rot / 2) it is read
  // from the row again and normed alike (all of them before anything is stored: out may be x)
  float oth[HNR_MAX_E];
  const int hr = rot >> 1;
#pragma unroll
  for (int e = 0; e < HNR_MAX_E; ++e) {
    const int c = lane + 64 * e;
    oth[e] = __shfl_xor(v[e], 1, 64);
    if (half && c < rot) {
      const int pc = c >= hr ? c - hr : c + hr;
      oth[e] = ldf(xr, pc) * (w != nullptr ? rs_w * w[pc] : 1.f);
    }
  }
#pragma unroll
  for (int e = 0; e < HNR_MAX_E; ++e) {
    const int c = lane + 64 * e;
    float val = v[e];
    if (c < rot) {
      const bool second = half ? c >= hr : (c & 1);
      const int fi = half ? (second ? c - hr : c) : (c >> 1);
      const float ang = pos * freqs[fi];
      const float cs = amp * cosf(ang), sn = amp * sinf(ang);
      val = second ? v[e] * cs + oth[e] * sn : v[e] * cs - oth[e] * sn;
    }
    if (!unit_after) { if (c < n) stf(orow, c, val); }
    else v[e] = val;
  }
  if (unit_after) {                                  // (block-uniform)
    float s2 = 0.f;
#pragma unroll
    for (int e = 0; e < HNR_MAX_E; ++e) s2 += v[e] * v[e];          // (entries past n are zeros)
    const float rs = 1.f / sqrtf(wave_sum(s2) / (float)n + eps);
#pragma unroll
    for (int e = 0; e < HNR_MAX_E; ++e) { const int c = lane + 64 * e; if (c < n) stf(orow, c, v[e] * rs); }
  }
}

extern "C" int fls_seq_head_norm_rope(const void* x, int tx, int ldx, int x_col, int x_hs, int heads, int n, const float* w,
                                      float eps, const float* freqs, int rot, const int* tok_pos, const int* row_map, void* out,
                                      int to, int ldo, int out_col, int out_hs, void* raw, int ldr, int rows, int unit_after,
                                      int half, float amp, fls_stream_t s) {
  if (rows <= 0 || heads <= 0) return 0;
  if (n < 1 || n > 64 * HNR_MAX_E || rot < 0 || rot > n || (rot & 1) || (rot > 0 && (freqs == nullptr || tok_pos == nullptr))) return -1;
  const int items = rows * heads;
  dim3 grid((items + 3) / 4);
  hipStream_t st = (hipStream_t)s;
#define HNR(TI, TO) hipLaunchKernelGGL((head_norm_rope_kernel<TI, TO>), grid, dim3(256), 0, st, (const TI*)x, ldx, x_col, x_hs, heads, \
                                       n, w, eps, freqs, rot, tok_pos, row_map, (TO*)out, ldo, out_col, out_hs, (TO*)raw, ldr, items, unit_after, half, amp)
  if (tx == 1 && to == 1) HNR(bf16_t, bf16_t);
  else if (tx == 1) HNR(bf16_t, float);
  else if (to == 1) HNR(float, bf16_t);
  else HNR(float, float);
#undef HNR
  SEQ_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------------ mixture of experts
// one thread per token: softmax statistics, then `top` passes each taking the best unchosen expert.
// corr == null: the `top` largest logits are chosen (ties: the lower expert) and weighted by the softmax
// over the chosen logits only
#define MOE_MAX_TOP 16
__global__ void moe_route_kernel(const float* __restrict__ logits, int ldl, const float* __restrict__ corr, int T, int E, int top,
                                 int* __restrict__ ids, float* __restrict__ w, int* __restrict__ hist) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  const float* l = logits + (size_t)t * ldl;
  if (corr == nullptr) {
    int chosen[MOE_MAX_TOP];
    float val[MOE_MAX_TOP];
    for (int k = 0; k < top; ++k) {
      float best = -INFINITY;
      int be = -1;
      for (int e = 0; e < E; ++e) {
        bool used = false;
        for (int j = 0; j < k; ++j) used |= (chosen[j] == e);
        if (used) continue;
        const float c = l[e];
        if (be < 0 || c > best) { best = c; be = e; }
      }
      chosen[k] = be;
      val[k] = best;
    }
    const float mx = val[0];                          // (the first choice is the largest)
    float sum = 0.f;
    for (int k = 0; k < top; ++k) { val[k] = expf(val[k] - mx); sum += val[k]; }
    const float inv = 1.f / sum;
    for (int k = 0; k < top; ++k) {
      ids[(size_t)t * top + k] = chosen[k];
      w[(size_t)t * top + k] = val[k] * inv;
    }
    return;
  }
  float mx = -INFINITY;
  for (int e = 0; e < E; ++e) mx = fmaxf(mx, l[e]);
  float sum = 0.f;
  for (int e = 0; e < E; ++e) sum += expf(l[e] - mx);
  const float inv = 1.f / sum;
  int chosen[MOE_MAX_TOP];
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY, bs = 0.f;
    int be = 0;
    for (int e = 0; e < E; ++e) {
      bool used = false;
      for (int j = 0; j < k; ++j) used |= (chosen[j] == e);
      if (used) continue;
      const float sc = expf(l[e] - mx) * inv;
      const float c = sc + corr[e];
      if (c > best) { best = c; be = e; bs = sc; }
    }
    chosen[k] = be;
    ids[(size_t)t * top + k] = be;
    w[(size_t)t * top + k] = bs;
  }
}

// entries per expert: a block counts its entries in LDS, then adds one number per expert to hist
#define MOE_MAX_E 1024
__global__ __launch_bounds__(256) void moe_hist_kernel(const int* __restrict__ ids, int n, int E, int* __restrict__ hist) {
  __shared__ int h[MOE_MAX_E];
  for (int e = threadIdx.x; e < E; e += 256) h[e] = 0;
  __syncthreads();
  for (int i = blockIdx.x * 4096 + threadIdx.x; i < min(n, (int)(blockIdx.x + 1) * 4096); i += 256) atomicAdd(&h[ids[i]], 1);
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += 256)
    if (h[e]) atomicAdd(hist + e, h[e]);
}

// one thread per token: scores sigmoid(logit); the experts form `groups` equal groups of neighbours, a group is worth the
// sum of its two largest scores, only experts of the `keep` best groups compete (ties: the lower group / expert);
// weights = score / (sum of the chosen + 1e-20) * scale.  groups <= 1: every expert competes
#define MOE_MAX_GROUPS 64
__global__ void moe_route_grouped_kernel(const float* __restrict__ logits, int ldl, int T, int E, int top, int groups, int keep,
                                         float scale, int* __restrict__ ids, float* __restrict__ w) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  const float* l = logits + (size_t)t * ldl;
  unsigned long long kept = ~0ull;
  const int per = groups > 1 ? E / groups : E;
  if (groups > 1) {
    float worth[MOE_MAX_GROUPS];
    for (int g = 0; g < groups; ++g) {
      float b1 = -1.f, b2 = -1.f;                     // (scores lie in (0, 1))
      for (int e = g * per; e < (g + 1) * per; ++e) {
        const float sc = sigmoid_f(l[e]);
        if (sc > b1) { b2 = b1; b1 = sc; } else if (sc > b2) { b2 = sc; }
      }
      worth[g] = b1 + (b2 > 0.f ? b2 : 0.f);
    }
    kept = 0ull;
    for (int k = 0; k < keep; ++k) {
      float best = -1.f;
      int bg = 0;
      for (int g = 0; g < groups; ++g)
        if (!((kept >> g) & 1ull) && worth[g] > best) { best = worth[g]; bg = g; }
      kept |= 1ull << bg;
    }
  }
  int chosen[MOE_MAX_TOP];
  float val[MOE_MAX_TOP];
  float sum = 0.f;
  for (int k = 0; k < top; ++k) {
    float best = -1.f;
    int be = 0;
    for (int e = 0; e < E; ++e) {
      if (groups > 1 && !((kept >> (e / per)) & 1ull)) continue;
      bool used = false;
      for (int j = 0; j < k; ++j) used |= (chosen[j] == e);
      if (used) continue;
      const float sc = sigmoid_f(l[e]);
      if (sc > best) { best = sc; be = e; }
    }
    chosen[k] = be;
    val[k] = best;
    sum += best;
  }
  const float inv = scale / (sum + 1e-20f);
  for (int k = 0; k < top; ++k) {
    ids[(size_t)t * top + k] = chosen[k];
    w[(size_t)t * top + k] = val[k] * inv;
  }
}

extern "C" int fls_seq_moe_route_grouped(const float* logits, int ldl, int T, int E, int top, int groups, int keep, float scale,
                                         int* ids, float* w, int* hist, fls_stream_t s) {
  if (T <= 0) return 0;
  if (top < 1 || top > MOE_MAX_TOP || top > E || E > MOE_MAX_E || groups < 0 || groups > MOE_MAX_GROUPS) return -1;
  if (groups > 1 && (E % groups || keep < 1 || keep > groups || keep * (E / groups) < top)) return -1;
  hipLaunchKernelGGL(moe_route_grouped_kernel, dim3((T + 127) / 128), dim3(128), 0, (hipStream_t)s, logits, ldl, T, E, top, groups,
                     keep, scale, ids, w);
  SEQ_LAUNCH_CHECK();
  hipLaunchKernelGGL(moe_hist_kernel, dim3((T * top + 4095) / 4096), dim3(256), 0, (hipStream_t)s, ids, T * top, E, hist);
  SEQ_LAUNCH_CHECK();
  return 0;
}

extern "C" int fls_seq_moe_route(const float* logits, int ldl, const float* corr, int T, int E, int top, int* ids, float* w,
                                 int* hist, fls_stream_t s) {
  if (T <= 0) return 0;
  if (top < 1 || top > MOE_MAX_TOP || top > E || E > MOE_MAX_E) return -1;
  hipLaunchKernelGGL(moe_route_kernel, dim3((T + 127) / 128), dim3(128), 0, (hipStream_t)s, logits, ldl, corr, T, E, top, ids, w, hist);
  SEQ_LAUNCH_CHECK();
  hipLaunchKernelGGL(moe_hist_kernel, dim3((T * top + 4095) / 4096), dim3(256), 0, (hipStream_t)s, ids, T * top, E, hist);
  SEQ_LAUNCH_CHECK();
  return 0;
}

__global__ void moe_scan_kernel(const int* __restrict__ hist, int E, int* __restrict__ offs, int* __restrict__ cursor) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    int acc = 0;
    for (int e = 0; e < E; ++e) { offs[e] = acc; cursor[e] = acc; acc += hist[e]; }
    offs[E] = acc;
  }
}

extern "C" int fls_seq_moe_scan(const int* hist, int E, int* offs, int* cursor, fls_stream_t s) {
  hipLaunchKernelGGL(moe_scan_kernel, dim3(1), dim3(64), 0, (hipStream_t)s, hist, E, offs, cursor);
  SEQ_LAUNCH_CHECK();
  return 0;
}

__global__ void moe_place_kernel(const int* __restrict__ ids, int n, int top, int* __restrict__ cursor, int* __restrict__ dest,
                                 int* __restrict__ rows) {
  // the lanes of a wave that go to the same expert take their places with one atomic: the first of
  // them adds their count to the expert's cursor, each takes base + its rank among them
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  const bool valid = i < n;
  const int e = valid ? ids[i] : -1;
  const int lane = threadIdx.x & 63;
  unsigned long long todo = __ballot(valid);
  while (todo) {
    const int leader = __ffsll((long long)todo) - 1;
    const int el = __shfl(e, leader, 64);
    const unsigned long long same = __ballot(valid && e == el);
    int base = 0;
    if (lane == leader) base = atomicAdd(cursor + el, __popcll(same));
    base = __shfl(base, leader, 64);
    if (valid && e == el) {
      const int p = base + __popcll(same & ((1ull << lane) - 1ull));
      dest[i] = p;
      rows[p] = i / top;
    }
    todo &= ~same;
  }
}

extern "C" int fls_seq_moe_place(const int* ids, int n, int top, int* cursor, int* dest, int* rows, fls_stream_t s) {
  if (n <= 0) return 0;
  hipLaunchKernelGGL(moe_place_kernel, dim3((n + 255) / 256), dim3(256), 0, (hipStream_t)s, ids, n, top, cursor, dest, rows);
  SEQ_LAUNCH_CHECK();
  return 0;
}

__global__ void moe_sum_kernel(const float* __restrict__ y, int ldy, const int* __restrict__ dest, const float* __restrict__ w,
                               float* __restrict__ out, int ldo, int top, int D) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < D; c += blockDim.x) {
    float acc = 0.f;
    for (int k = 0; k < top; ++k) acc += w[(size_t)t * top + k] * y[(size_t)dest[(size_t)t * top + k] * ldy + c];
    out[(size_t)t * ldo + c] = acc;
  }
}

extern "C" int fls_seq_moe_sum(const float* y, int ldy, const int* dest, const float* w, float* out, int ldo, int T, int top,
                               int D, fls_stream_t s) {
  if (T <= 0) return 0;
  hipLaunchKernelGGL(moe_sum_kernel, dim3(T), dim3(256), 0, (hipStream_t)s, y, ldy, dest, w, out, ldo, top, D);
  SEQ_LAUNCH_CHECK();
  return 0;
}

// x[t, c] += mult * (sum_k w[t, k] y[dest[t, k], c] + sigmoid(gate[t]) shared[t, c]); shared / gate nullable
__global__ __launch_bounds__(256) void moe_combine_kernel(float* __restrict__ x, int ldx, const float* __restrict__ y, int ldy,
                                                          const int* __restrict__ dest, const float* __restrict__ w, int top,
                                                          const float* __restrict__ shared, int lds, const float* __restrict__ gate,
                                                          int ldg, int D, float mult) {
  const int t = blockIdx.x;
  const float sg = shared == nullptr ? 0.f : (gate != nullptr ? sigmoid_f(gate[(size_t)t * ldg]) : 1.f);
  for (int c = blockIdx.y * 256 + threadIdx.x; c < D; c += 256 * gridDim.y) {
    float acc = 0.f;
    for (int k = 0; k < top; ++k) acc += w[(size_t)t * top + k] * y[(size_t)dest[(size_t)t * top + k] * ldy + c];
    if (shared != nullptr) acc += sg * shared[(size_t)t * lds + c];
    x[(size_t)t * ldx + c] += mult * acc;
  }
}

extern "C" int fls_seq_moe_combine(float* x, int ldx, const float* y, int ldy, const int* dest, const float* w, int T, int top,
                                   const float* shared, int lds, const float* gate, int ldg, int D, float mult, fls_stream_t s) {
  if (T <= 0) return 0;
  hipLaunchKernelGGL(moe_combine_kernel, dim3(T, (D + 1023) / 1024), dim3(256), 0, (hipStream_t)s, x, ldx, y, ldy, dest, w, top, shared,
                     lds, gate, ldg, D, mult);
  SEQ_LAUNCH_CHECK();
  return 0;
}

extern "C" int fls_seq_version(void) { return 10; }
