// Several residual streams per row (hyper-connections), the gated residual update, differential
// attention's combine, and small row kernels beside them.  A row's S streams lie side by side:
// xs[t, s * D + c].  Everything is fp32 except the rows handed to the next matrix product.
#include "seq_common.h"
#include "fls_seq.h"

#define MAX_STREAMS 8

// ------------------------------------------------------------------------------- embedding
// out[t, c * D + j] = table[ids[t], j] * scale + pos_table[tok_pos[t], j] for every copy c
template <typename T>
__global__ void embed_pos_kernel(const int* __restrict__ ids, const T* __restrict__ table, const T* __restrict__ pos_table,
                                 const int* __restrict__ tok_pos, float* __restrict__ out, int D, int V, int P, float scale,
                                 int copies) {
  const int t = blockIdx.x;
  int id = ids[t];
  id = id < 0 ? 0 : (id >= V ? V - 1 : id);
  const T* row = table + (size_t)id * D;
  const T* prow = nullptr;
  if (pos_table != nullptr) {
    int p = tok_pos[t];
    p = p < 0 ? 0 : (p >= P ? P - 1 : p);
    prow = pos_table + (size_t)p * D;
  }
  float* o = out + (size_t)t * D * copies;
  for (int j = threadIdx.x; j < D; j += blockDim.x) {
    float v = ldf(row, j) * scale;
    if (prow != nullptr) v += ldf(prow, j);
    for (int c = 0; c < copies; ++c) o[(size_t)c * D + j] = v;
  }
}

extern "C" int fls_seq_embed_pos(const int* ids, const void* table, int tt, const void* pos_table, const int* tok_pos, float* out,
                                 int T, int D, int V, int P, float scale, int copies, fls_stream_t s) {
  if (T <= 0) return 0;
  if (copies < 1 || (pos_table != nullptr && (tok_pos == nullptr || P < 1))) return -1;
  if (tt == 1) hipLaunchKernelGGL((embed_pos_kernel<bf16_t>), dim3(T), dim3(256), 0, (hipStream_t)s, ids, (const bf16_t*)table,
                                  (const bf16_t*)pos_table, tok_pos, out, D, V, P, scale, copies);
  else hipLaunchKernelGGL((embed_pos_kernel<float>), dim3(T), dim3(256), 0, (hipStream_t)s, ids, (const float*)table,
                          (const float*)pos_table, tok_pos, out, D, V, P, scale, copies);
  SEQ_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------------ streams -> normed row
// one block per row: u = sum_s coef[s] xs_s (kept in registers, four columns a thread per 1024-column piece),
// block sum of u^2, y = u rs w
#define SN_PIECES 8                // columns <= 8192 stay in registers; wider rows are read twice
template <typename TO>
__global__ __launch_bounds__(256) void streams_norm_kernel(const float* __restrict__ xs, int ldx, const int* __restrict__ idx,
                                                           const float* __restrict__ coef, const float* __restrict__ w,
                                                           TO* __restrict__ y, int ldy, int D, int S, float eps) {
  __shared__ float red[4];
  const int r = blockIdx.x;
  const float* xr = xs + (size_t)(idx != nullptr ? idx[r] : r) * ldx;
  float cf[MAX_STREAMS];
#pragma unroll
  for (int s = 0; s < MAX_STREAMS; ++s) cf[s] = s < S ? (coef != nullptr ? coef[s] : 1.f) : 0.f;
  float u[SN_PIECES];
  float ss = 0.f;
  const bool fits = D <= 256 * SN_PIECES;
  if (fits) {
#pragma unroll
    for (int k = 0; k < SN_PIECES; ++k) {
      const int c = threadIdx.x + 256 * k;
      float a = 0.f;
      if (c < D)
        for (int s = 0; s < S; ++s) a += cf[s] * xr[(size_t)s * D + c];
      u[k] = a;
      ss += a * a;
    }
  } else {
    for (int c = threadIdx.x; c < D; c += 256) {
      float a = 0.f;
      for (int s = 0; s < S; ++s) a += cf[s] * xr[(size_t)s * D + c];
      ss += a * a;
    }
  }
  ss = block_sum_256(ss, red);
  const float rs = 1.f / sqrtf(ss / (float)D + eps);
  TO* yr = y + (size_t)r * ldy;
  if (fits) {
#pragma unroll
    for (int k = 0; k < SN_PIECES; ++k) {
      const int c = threadIdx.x + 256 * k;
      if (c < D) stf(yr, c, u[k] * rs * w[c]);
    }
  } else {
    for (int c = threadIdx.x; c < D; c += 256) {
      float a = 0.f;
      for (int s = 0; s < S; ++s) a += cf[s] * xr[(size_t)s * D + c];
      stf(yr, c, a * rs * w[c]);
    }
  }
}

extern "C" int fls_seq_streams_norm(const float* xs, int ldx, const int* idx, const float* coef, const float* w, void* y, int ty,
                                    int ldy, int rows, int D, int S, float eps, fls_stream_t s) {
  if (rows <= 0) return 0;
  if (S < 1 || S > MAX_STREAMS || ldx < S * D) return -1;
  hipStream_t st = (hipStream_t)s;
  if (ty == 1) hipLaunchKernelGGL((streams_norm_kernel<bf16_t>), dim3(rows), dim3(256), 0, st, xs, ldx, idx, coef, w, (bf16_t*)y, ldy, D, S, eps);
  else hipLaunchKernelGGL((streams_norm_kernel<float>), dim3(rows), dim3(256), 0, st, xs, ldx, idx, coef, w, (float*)y, ldy, D, S, eps);
  SEQ_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------------ streams update (+ next norm)
// one block per row.  Per column: the S old values, the gated sublayer output g = y sigmoid(gate), the S new
// values mix^T old + mult out g, written back; with NORM also u = sum_s ncoef[s] new_s, whose norm is the next
// sublayer's input.  Columns <= 256 * SN_PIECES keep u in registers between the two halves.
template <typename TO, int NORM>
__global__ __launch_bounds__(256) void streams_update_kernel(float* __restrict__ xs, int ldx, const float* __restrict__ y, int ldy,
                                                             const float* __restrict__ gate, int ldg,
                                                             const float* __restrict__ hc, float mult, int D, int S,
                                                             const float* __restrict__ ncoef, const float* __restrict__ nw,
                                                             TO* __restrict__ h, int ldh, float eps) {
  __shared__ float red[4];
  __shared__ float mixs[MAX_STREAMS * MAX_STREAMS], outs[MAX_STREAMS], ncs[MAX_STREAMS];
  if (threadIdx.x < S * S) mixs[threadIdx.x] = hc != nullptr ? hc[2 * S + threadIdx.x] : 1.f;
  if (threadIdx.x < S) {
    outs[threadIdx.x] = mult * (hc != nullptr ? hc[S + threadIdx.x] : 1.f);
    ncs[threadIdx.x] = (NORM && ncoef != nullptr) ? ncoef[threadIdx.x] : 1.f;
  }
  __syncthreads();
  const int r = blockIdx.x;
  float* xr = xs + (size_t)r * ldx;
  const float* yr = y + (size_t)r * ldy;
  const float* gr = gate != nullptr ? gate + (size_t)r * ldg : nullptr;
  float u[SN_PIECES];
  float ss = 0.f;
  const int npieces = (D + 255) / 256;
  // one column: the old streams in, the new ones out; returns the column's entry of the next sublayer's input
  auto column = [&](int c) -> float {
    float old[MAX_STREAMS];
#pragma unroll
    for (int s = 0; s < MAX_STREAMS; ++s) old[s] = s < S ? xr[(size_t)s * D + c] : 0.f;
    float g = yr[c];
    if (gr != nullptr) g *= sigmoid_f(gr[c]);
    float un = 0.f;
#pragma unroll
    for (int t = 0; t < MAX_STREAMS; ++t) {
      if (t < S) {
        float v = outs[t] * g;
#pragma unroll
        for (int s = 0; s < MAX_STREAMS; ++s)
          if (s < S) v += mixs[s * S + t] * old[s];
        xr[(size_t)t * D + c] = v;
        un += ncs[t] * v;
      }
    }
    return un;
  };
#pragma unroll
  for (int k = 0; k < SN_PIECES; ++k) {
    const int c = threadIdx.x + 256 * k;
    u[k] = c < D ? column(c) : 0.f;
    ss += u[k] * u[k];
  }
  for (int k = SN_PIECES; k < npieces; ++k) {
    const int c = threadIdx.x + 256 * k;
    if (c < D) { const float un = column(c); ss += un * un; }
  }
  if (!NORM) return;
  ss = block_sum_256(ss, red);
  const float rs = 1.f / sqrtf(ss / (float)D + eps);
  TO* hr = h + (size_t)r * ldh;
#pragma unroll
  for (int k = 0; k < SN_PIECES; ++k) {
    const int c = threadIdx.x + 256 * k;
    if (c < D) stf(hr, c, u[k] * rs * nw[c]);
  }
  for (int k = SN_PIECES; k < npieces; ++k) {    // (a thread re-reads only what it wrote itself)
    const int c = threadIdx.x + 256 * k;
    if (c >= D) break;
    float un = 0.f;
    for (int t = 0; t < S; ++t) un += ncs[t] * xr[(size_t)t * D + c];
    stf(hr, c, un * rs * nw[c]);
  }
}

extern "C" int fls_seq_streams_update(float* xs, int ldx, const float* y, int ldy, const float* gate, int ldg, const float* hc,
                                      float mult, int rows, int D, int S, const float* ncoef, const float* nw, void* h, int th,
                                      int ldh, float eps, fls_stream_t s) {
  if (rows <= 0) return 0;
  if (S < 1 || S > MAX_STREAMS || ldx < S * D || (hc == nullptr && S != 1) || (h != nullptr && nw == nullptr)) return -1;
  hipStream_t st = (hipStream_t)s;
#define SU(TO, N) hipLaunchKernelGGL((streams_update_kernel<TO, N>), dim3(rows), dim3(256), 0, st, xs, ldx, y, ldy, gate, ldg, hc, mult, \
                                     D, S, ncoef, nw, (TO*)h, ldh, eps)
  if (h == nullptr) SU(float, 0);
  else if (th == 1) SU(bf16_t, 1);
  else SU(float, 1);
#undef SU
  SEQ_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------------------- small row kernels
__global__ void scale_kernel(float* __restrict__ z, int ldz, int cols, float alpha) {
  float* zr = z + (size_t)blockIdx.x * ldz;
  for (int c = threadIdx.x; c < cols; c += blockDim.x) zr[c] *= alpha;
}

extern "C" int fls_seq_scale(float* z, int ldz, int rows, int cols, float alpha, fls_stream_t s) {
  if (rows <= 0) return 0;
  hipLaunchKernelGGL(scale_kernel, dim3(rows), dim3(256), 0, (hipStream_t)s, z, ldz, cols, alpha);
  SEQ_LAUNCH_CHECK();
  return 0;
}

template <typename TI, typename TO>
__global__ void sigmoid_gate_kernel(const TI* __restrict__ o, int ldo, const float* __restrict__ g, int ldg, TO* __restrict__ y,
                                    int ldy, int cols) {
  const TI* orow = o + (size_t)blockIdx.x * ldo;
  const float* gr = g + (size_t)blockIdx.x * ldg;
  TO* yr = y + (size_t)blockIdx.x * ldy;
  for (int c = threadIdx.x; c < cols; c += blockDim.x) stf(yr, c, ldf(orow, c) * sigmoid_f(gr[c]));
}

extern "C" int fls_seq_sigmoid_gate(const void* o, int to_, int ldo, const float* g, int ldg, void* y, int ty, int ldy, int rows,
                                    int cols, fls_stream_t s) {
  if (rows <= 0) return 0;
  hipStream_t st = (hipStream_t)s;
#define SG(TI, TO) hipLaunchKernelGGL((sigmoid_gate_kernel<TI, TO>), dim3(rows), dim3(256), 0, st, (const TI*)o, ldo, g, ldg, (TO*)y, ldy, cols)
  if (to_ == 1 && ty == 1) SG(bf16_t, bf16_t);
  else if (to_ == 1) SG(bf16_t, float);
  else if (ty == 1) SG(float, bf16_t);
  else SG(float, float);
#undef SG
  SEQ_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------------ differential attention's combine
// one wave per (row, head): o = a1 - lambda a2 over the head's dv columns (up to 8 a lane), wave sum of o^2,
// out = o / sqrt(mean(o^2) + eps) (1 - diff).  lambda from lam_w [4, d]: every wave works it out for itself.
template <typename TO>
__global__ __launch_bounds__(256) void diff_combine_kernel(const float* __restrict__ a, int lda, const float* __restrict__ lam_w,
                                                           int d, float diff, int H, int dv, float eps, TO* __restrict__ out,
                                                           int ldo, int items) {
  const int lane = threadIdx.x & 63;
  const int item = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= items) return;
  const int t = item / H, h = item % H;
  float s1 = 0.f, s2 = 0.f;
  for (int c = lane; c < d; c += 64) { s1 += lam_w[c] * lam_w[d + c]; s2 += lam_w[2 * d + c] * lam_w[3 * d + c]; }
  const float lam = expf(wave_sum(s1)) - expf(wave_sum(s2)) + diff;
  const float* a1 = a + (size_t)t * lda + (size_t)h * dv;
  const float* a2 = a1 + (size_t)H * dv;
  float o[8];
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int c = lane + 64 * e;
    o[e] = c < dv ? a1[c] - lam * a2[c] : 0.f;
    ss += o[e] * o[e];
  }
  const float rs = (1.f - diff) / sqrtf(wave_sum(ss) / (float)dv + eps);
  TO* orow = out + (size_t)t * ldo + (size_t)h * dv;
#pragma unroll
  for (int e = 0; e < 8; ++e) { const int c = lane + 64 * e; if (c < dv) stf(orow, c, o[e] * rs); }
}

extern "C" int fls_seq_diff_combine(const float* a, int lda, const float* lam_w, int d, float diff, int H, int dv, float eps,
                                    void* out, int to, int ldo, int T, fls_stream_t s) {
  if (T <= 0) return 0;
  if (dv < 1 || dv > 512 || H < 1 || d < 1 || lda < 2 * H * dv) return -1;
  const int items = T * H;
  hipStream_t st = (hipStream_t)s;
  if (to == 1) hipLaunchKernelGGL((diff_combine_kernel<bf16_t>), dim3((items + 3) / 4), dim3(256), 0, st, a, lda, lam_w, d, diff, H, dv, eps, (bf16_t*)out, ldo, items);
  else hipLaunchKernelGGL((diff_combine_kernel<float>), dim3((items + 3) / 4), dim3(256), 0, st, a, lda, lam_w, d, diff, H, dv, eps, (float*)out, ldo, items);
  SEQ_LAUNCH_CHECK();
  return 0;
}
