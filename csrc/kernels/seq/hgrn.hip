// HGRN2: a gated linear recurrence whose forget gate also sets what is written.  Per head a state
// S [d, dv] in fp32:  S_t = diag(g_t) S_(t-1) + (1 - g_t) v_t^T,  o_t = S_t^T silu(q_t),
// g = lower + (1 - lower) sigmoid(f (+ fb)).
//
// block = (tile of value columns, head, request).  A value column's d state rows are cut over NS lanes
// (HG_NPT rows each, in registers); the block walks the request's rows in order, HG_TT rows at a time: their
// gates (sigmoid and lower bound applied), silu(q) and v are staged in LDS by all threads, then every lane
// updates its rows and the NS lanes of a column add their parts of o by shuffles.  The raw o goes to an fp32
// matrix; the per-head RMS norm runs afterwards over whole heads (a head's columns may span several blocks).
#include "seq_common.h"
#include "fls_seq.h"

#define HG_NPT 16
#define HG_TT 16
template <int NS>
__global__ __launch_bounds__(256) void hgrn2_scan_kernel(const float* __restrict__ q, int ldq, const float* __restrict__ f, int ldf,
                                                         const float* __restrict__ v, int ldv, const float* __restrict__ fb,
                                                         const float* __restrict__ lower, float* __restrict__ state,
                                                         float* __restrict__ out, int ldo, const int* __restrict__ cu,
                                                         const int* __restrict__ pos0, const int* __restrict__ slot, int H, int d,
                                                         int dv) {
  constexpr int PPB = 256 / NS;                    // value columns per block
  constexpr int NMAX = NS * HG_NPT;                // state rows the lanes of a column cover
  __shared__ float gs[HG_TT][NMAX], qs[HG_TT][NMAX];
  __shared__ float vs[HG_TT][PPB];
  const int s = blockIdx.z, h = blockIdx.y;
  const int ns = threadIdx.x % NS, pl = threadIdx.x / NS;
  const int p0 = blockIdx.x * PPB;
  const int p = p0 + pl;
  const bool live = p < dv;
  const int a0 = cu[s], a1 = cu[s + 1];
  float S[HG_NPT];
  float* sp = state + (((size_t)slot[s] * H + h) * d) * dv + (live ? p : 0);
  const bool carried = pos0[s] > 0;
#pragma unroll
  for (int i = 0; i < HG_NPT; ++i) {
    const int n = i * NS + ns;
    S[i] = (carried && live && n < d) ? sp[(size_t)n * dv] : 0.f;
  }
  for (int t0 = a0; t0 < a1; t0 += HG_TT) {
    const int nt = min(HG_TT, a1 - t0);
    __syncthreads();
    for (int e = threadIdx.x; e < nt * NMAX; e += 256) {
      const int tt = e / NMAX, n = e % NMAX;
      float g = 1.f, qv = 0.f;                     // (rows past d: state stays zero, contributes nothing)
      if (n < d) {
        const int c = h * d + n;
        const float lo = lower[c];
        float z = f[(size_t)(t0 + tt) * ldf + c];
        if (fb != nullptr) z += fb[c];
        g = lo + (1.f - lo) * sigmoid_f(z);
        qv = silu_f(q[(size_t)(t0 + tt) * ldq + c]);
      }
      gs[tt][n] = g;
      qs[tt][n] = qv;
    }
    for (int e = threadIdx.x; e < nt * PPB; e += 256) {
      const int tt = e / PPB, c = e % PPB;
      vs[tt][c] = p0 + c < dv ? v[(size_t)(t0 + tt) * ldv + h * dv + p0 + c] : 0.f;
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float vv = vs[tt][pl];
      float yv = 0.f;
#pragma unroll
      for (int i = 0; i < HG_NPT; ++i) {
        const int n = i * NS + ns;
        const float g = gs[tt][n];
        S[i] = g * S[i] + (1.f - g) * vv;
        yv += S[i] * qs[tt][n];
      }
#pragma unroll
      for (int o = NS / 2; o > 0; o >>= 1) yv += __shfl_xor(yv, o, 64);
      if (ns == 0 && live) out[(size_t)(t0 + tt) * ldo + h * dv + p] = yv;
    }
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < HG_NPT; ++i) {
      const int n = i * NS + ns;
      if (n < d) sp[(size_t)n * dv] = S[i];
    }
  }
}

// raw: fp32 [T, H dv] with row stride ldo, the un-normed outputs
extern "C" int fls_seq_hgrn2_scan(const float* q, int ldq, const float* f, int ldf, const float* v, int ldv, const float* fb,
                                  const float* lower, float* state, float* raw, int ldo, const int* cu, const int* pos0,
                                  const int* slot, int B, int H, int d, int dv, fls_stream_t s) {
  if (B <= 0) return 0;
  if (d < 1 || d > 256 || dv < 1 || H < 1) return -1;
  int nsl = 1;
  while (nsl * HG_NPT < d) nsl *= 2;
  hipStream_t st = (hipStream_t)s;
#define HG_LAUNCH(NSV) hipLaunchKernelGGL((hgrn2_scan_kernel<NSV>), dim3((dv + 256 / NSV - 1) / (256 / NSV), H, B), dim3(256), 0, st, \
    q, ldq, f, ldf, v, ldv, fb, lower, state, raw, ldo, cu, pos0, slot, H, d, dv)
  switch (nsl) {
    case 1: HG_LAUNCH(1); break;
    case 2: HG_LAUNCH(2); break;
    case 4: HG_LAUNCH(4); break;
    case 8: HG_LAUNCH(8); break;
    default: HG_LAUNCH(16); break;
  }
#undef HG_LAUNCH
  SEQ_LAUNCH_CHECK();
  return 0;
}
