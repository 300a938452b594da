// Recurrent mixers of the stateful models: the short causal convolution with its carried inputs, the
// gated linear recurrence (RG-LRU) and the selective state-space scan (Mamba-2 form).  States are
// fp32 and live in slots; a request whose step starts at position 0 starts from zeros without
// reading its slot, so slots are never cleared.  Every kernel walks a request's rows of this step
// in order, whatever their number: a whole prompt, a portion of one, or one decoded token.
#include "seq_common.h"
#include "fls_seq.h"

// ------------------------------------------------------------------------ causal convolution
// out[t, c] = b[c] + sum_j w[c, taps-1-j] * in(t - j) (+ in(t) when residual; b may be null); in() before this
// step's first row comes from state[slot] (the last taps-1 inputs of the request), zeros before position 0.
// act: 1 = silu.  The sum is fp32; the output has the type the consumer reads.
template <typename TO>
__global__ void causal_conv_kernel(const float* __restrict__ x, int ldx, const float* __restrict__ w, const float* __restrict__ b,
                                   const float* __restrict__ state, TO* __restrict__ out, int ldo,
                                   const int* __restrict__ tok_seq, const int* __restrict__ cu, const int* __restrict__ pos0,
                                   const int* __restrict__ slot, int C, int taps, int act, int residual) {
  const int t = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int s = tok_seq[t];
  const int tl = t - cu[s];
  const bool carried = pos0[s] > 0;
  const float* hist = state + (size_t)slot[s] * (taps - 1) * C;
  float acc = b != nullptr ? b[c] : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int src = tl - j;
    float v = 0.f;
    if (src >= 0) v = x[(size_t)(t - j) * ldx + c];
    else if (carried) v = hist[(size_t)(taps - 1 + src) * C + c];
    acc += w[(size_t)c * taps + (taps - 1 - j)] * v;
  }
  if (residual) acc += x[(size_t)t * ldx + c];
  stf(out + (size_t)t * ldo, c, act == 1 ? silu_f(acc) : acc);
}

// The same for up to CONV_MAX_TAPS taps with every input row read once: a thread owns a channel and
// walks CONV_ROWS consecutive rows, keeping the last taps inputs in registers (xv[j] = the input j rows
// back); only the first row of its run, or of a new request inside it, gathers its lags from memory or
// from the carried state.  fuse_state (every request of the step has one row, so the thread that walks a
// request's row has seen all its inputs): the thread also rewrites its channel of the carried state.
#define CONV_MAX_TAPS 8
#define CONV_ROWS 16
template <typename TO>
__global__ void causal_conv_rows_kernel(const float* __restrict__ x, int ldx, const float* __restrict__ w, const float* __restrict__ b,
                                        float* __restrict__ state, TO* __restrict__ out, int ldo,
                                        const int* __restrict__ tok_seq, const int* __restrict__ cu, const int* __restrict__ pos0,
                                        const int* __restrict__ slot, int T, int C, int taps, int act, int residual, int fuse_state) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int t0 = blockIdx.y * CONV_ROWS, t1 = min(T, t0 + CONV_ROWS);
  float wv[CONV_MAX_TAPS], xv[CONV_MAX_TAPS];
#pragma unroll
  for (int j = 0; j < CONV_MAX_TAPS; ++j) {
    wv[j] = j < taps ? w[(size_t)c * taps + (taps - 1 - j)] : 0.f;      // the weight of the input j rows back
    xv[j] = 0.f;
  }
  const float bias = b != nullptr ? b[c] : 0.f;
  int prev = -1;
  for (int t = t0; t < t1; ++t) {
    const int s = tok_seq[t];
    if (s != prev) {
      const int tl = t - cu[s];
      const bool carried = pos0[s] > 0;
      float* hist = state + (size_t)slot[s] * (taps - 1) * C;
#pragma unroll
      for (int j = 1; j < CONV_MAX_TAPS; ++j) {
        float v = 0.f;
        if (j < taps) {
          const int src = tl - j;
          if (src >= 0) v = x[(size_t)(t - j) * ldx + c];
          else if (carried) v = hist[(size_t)(taps - 1 + src) * C + c];
        }
        xv[j] = v;
      }
      prev = s;
      if (fuse_state) {                              // the request's only row: the state becomes its last taps - 1 inputs
        if (taps > 1) hist[(size_t)(taps - 2) * C + c] = x[(size_t)t * ldx + c];
#pragma unroll
        for (int j = 1; j < CONV_MAX_TAPS - 1; ++j)                        // the input j rows back moves to entry taps - 2 - j
          if (j <= taps - 2) hist[(size_t)(taps - 2 - j) * C + c] = xv[j];
      }
    } else {
#pragma unroll
      for (int j = CONV_MAX_TAPS - 1; j > 0; --j) xv[j] = xv[j - 1];
    }
    xv[0] = x[(size_t)t * ldx + c];
    float acc = bias;
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS; ++j) acc += wv[j] * xv[j];
    if (residual) acc += xv[0];
    stf(out + (size_t)t * ldo, c, act == 1 ? silu_f(acc) : acc);
  }
}

// the state after the step: the last taps-1 inputs.  One thread per (request, channel) walks the
// taps-1 entries upwards: entry k takes input n - (taps-1) + k of this step, or, when the step is
// shorter than the history, the old entry k + n, which no earlier iteration has overwritten.
__global__ void conv_state_kernel(const float* __restrict__ x, int ldx, float* __restrict__ state, const int* __restrict__ cu,
                                  const int* __restrict__ pos0, const int* __restrict__ slot, int C, int taps) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int a = cu[s], n = cu[s + 1] - a;
  const bool carried = pos0[s] > 0;
  float* hist = state + (size_t)slot[s] * (taps - 1) * C;
  for (int k = 0; k < taps - 1; ++k) {
    const int src = n - (taps - 1) + k;
    float v = 0.f;
    if (src >= 0) v = x[(size_t)(a + src) * ldx + c];
    else if (carried) v = hist[(size_t)(k + n) * C + c];
    hist[(size_t)k * C + c] = v;
  }
}

extern "C" int fls_seq_causal_conv(const float* x, int ldx, const float* w, const float* b, float* state, void* out, int to,
                                   int ldo, const int* tok_seq, const int* cu, const int* pos0, const int* slot, int T, int B,
                                   int C, int taps, int act, int residual, int one_row_each, fls_stream_t s) {
  if (T <= 0) return 0;
  if (taps < 1) return -1;
  hipStream_t st = (hipStream_t)s;
  if (taps <= CONV_MAX_TAPS) {
    dim3 grid((C + 255) / 256, (T + CONV_ROWS - 1) / CONV_ROWS);
    const int fuse = one_row_each && T == B;
    if (to == 1) hipLaunchKernelGGL((causal_conv_rows_kernel<bf16_t>), grid, dim3(256), 0, st, x, ldx, w, b, state, (bf16_t*)out, ldo, tok_seq, cu, pos0, slot, T, C, taps, act, residual, fuse);
    else hipLaunchKernelGGL((causal_conv_rows_kernel<float>), grid, dim3(256), 0, st, x, ldx, w, b, state, (float*)out, ldo, tok_seq, cu, pos0, slot, T, C, taps, act, residual, fuse);
    SEQ_LAUNCH_CHECK();
    if (fuse) return 0;
  } else if (to == 1) hipLaunchKernelGGL((causal_conv_kernel<bf16_t>), dim3((C + 255) / 256, T), dim3(256), 0, st, x, ldx, w, b, state, (bf16_t*)out, ldo, tok_seq, cu, pos0, slot, C, taps, act, residual);
  else hipLaunchKernelGGL((causal_conv_kernel<float>), dim3((C + 255) / 256, T), dim3(256), 0, st, x, ldx, w, b, state, (float*)out, ldo, tok_seq, cu, pos0, slot, C, taps, act, residual);
  SEQ_LAUNCH_CHECK();
  if (taps > 1) {
    hipLaunchKernelGGL(conv_state_kernel, dim3((C + 255) / 256, B), dim3(256), 0, st, x, ldx, state, cu, pos0, slot, C, taps);
    SEQ_LAUNCH_CHECK();
  }
  return 0;
}

// ------------------------------------------------ projected q | k | v rows on their way into attention
// z = [q (H d) | k (G d) | v (G dv) | ...] per row.  A wave serves heads of one row: a head's entries pass the causal
// convolution over the request's rows (w [C, taps], history from state[slot] as above; w null: none), then -- q and
// k heads -- the rotation of pairs (2i, 2i + 1) of the first `rot` entries by the angle pos * freqs[i] (the pair's
// other entry sits in the neighbouring lane) and the division by the head's root mean square (eps inside the
// root); q goes to qo[t] (fp32), k and v to row kv_slot[t] of their pools.  The angle depends on the row and the
// entry, not on the head, so a wave works out the sines and cosines of its lanes' entries once (full-range
// sincosf: angles reach thousands of radians) and walks several heads with them: block = (row, share of the
// row's heads), the four waves taking heads in turn; the host gives a row one block when rows are many and a wave
// per head when they are few.  fuse_state (every request brings one row): the wave also rewrites its channels of
// the carried history.  Head sizes <= 512.
// TAPS > 0: that many taps, all of a head's inputs and weights loaded before the sums (the loads of a head are
// in flight together); TAPS = 0: any number, or none.  NE: entries per lane (head sizes <= 64 NE).
#define QKV_MAX_E 8
template <typename TO, int TAPS, int NE>
__global__ __launch_bounds__(256) void qkv_conv_rope_kernel(const float* __restrict__ z, int ldz, const float* __restrict__ w,
                                                            float* __restrict__ state, int taps, const int* __restrict__ tok_seq,
                                                            const int* __restrict__ tok_pos, const int* __restrict__ cu,
                                                            const int* __restrict__ pos0, const int* __restrict__ slot,
                                                            const int* __restrict__ kv_slot, int H, int G, int d, int dv, float eps,
                                                            const float* __restrict__ freqs, int rot, float* __restrict__ qo,
                                                            int ldq, TO* __restrict__ kc, int ldk, TO* __restrict__ vc, int ldv,
                                                            int C, int fuse_state, int Gv, const float* __restrict__ qnw,
                                                            const float* __restrict__ knw) {
  const int lane = threadIdx.x & 63;
  const int t = blockIdx.x;
  const int ipr = H + G + Gv;
  const int s = tok_seq[t];
  const int tl = t - cu[s];
  const bool carried = pos0[s] > 0;
  float* hist = (w != nullptr && taps > 1) ? state + (size_t)slot[s] * (taps - 1) * C : nullptr;
  float cs[NE], sn[NE];
  {
    const float pos = rot > 0 ? (float)tok_pos[t] : 0.f;
#pragma unroll
    for (int e = 0; e < NE; ++e) {
      const int c = lane + 64 * e;
      cs[e] = 1.f;
      sn[e] = 0.f;
      if (c < rot) sincosf(pos * freqs[c >> 1], &sn[e], &cs[e]);
    }
  }
  for (int hi = blockIdx.y * 4 + (threadIdx.x >> 6); hi < ipr; hi += 4 * gridDim.y) {
    const int kind = hi < H ? 0 : (hi < H + G ? 1 : 2);
    const int n = kind == 2 ? dv : d;
    const int col0 = kind == 0 ? hi * d : (kind == 1 ? H * d + (hi - H) * d : (H + G) * d + (hi - H - G) * dv);
    float v[NE];
    if constexpr (TAPS > 0) {
      float in[NE][TAPS], wv[NE][TAPS];
#pragma unroll
      for (int e = 0; e < NE; ++e) {
        const int c = lane + 64 * e;
        const int ch = col0 + (c < n ? c : 0);
#pragma unroll
        for (int j = 0; j < TAPS; ++j) {
          const int src = tl - j;
          const float* p = src >= 0 ? z + (size_t)(t - j) * ldz + ch : (carried ? hist + (size_t)(TAPS - 1 + src) * C + ch : nullptr);
          in[e][j] = (p != nullptr && c < n) ? *p : 0.f;
          wv[e][j] = w[(size_t)ch * TAPS + (TAPS - 1 - j)];
        }
      }
#pragma unroll
      for (int e = 0; e < NE; ++e) {
        float acc = 0.f;
#pragma unroll
        for (int j = 0; j < TAPS; ++j) acc += wv[e][j] * in[e][j];
        v[e] = acc;
        const int c = lane + 64 * e;
        if (fuse_state && c < n) {                   // the request's only row: the history becomes its last TAPS - 1 inputs
          const int ch = col0 + c;
#pragma unroll
          for (int j = 0; j + 1 < TAPS; ++j) hist[(size_t)(TAPS - 2 - j) * C + ch] = in[e][j];
        }
      }
    } else {
#pragma unroll
      for (int e = 0; e < NE; ++e) {
        const int c = lane + 64 * e;
        float acc = 0.f;
        if (c < n) {
          const int ch = col0 + c;
          if (w == nullptr) {
            acc = z[(size_t)t * ldz + ch];
          } else {
            for (int j = 0; j < taps; ++j) {
              const int src = tl - j;
              float in = 0.f;
              if (src >= 0) in = z[(size_t)(t - j) * ldz + ch];
              else if (carried) in = hist[(size_t)(taps - 1 + src) * C + ch];
              acc += w[(size_t)ch * taps + (taps - 1 - j)] * in;
            }
            if (fuse_state && taps > 1) {            // the request's only row: shift the history, append this row
              for (int k = 0; k + 2 < taps; ++k) hist[(size_t)k * C + ch] = carried ? hist[(size_t)(k + 1) * C + ch] : 0.f;
              hist[(size_t)(taps - 2) * C + ch] = z[(size_t)t * ldz + ch];
            }
          }
        }
        v[e] = acc;
      }
    }
    if (kind == 2) {                                 // (wave-uniform)
      TO* vr = vc + (size_t)kv_slot[t] * ldv + (size_t)(hi - H - G) * dv;
#pragma unroll
      for (int e = 0; e < NE; ++e) { const int c = lane + 64 * e; if (c < n) stf(vr, c, v[e]); }
      continue;
    }
    float s2 = 0.f;
    // a weighted norm comes before the rotation: the root mean square of the entries as they are, the weight on every
    // entry, then the rotation (which the scalar 1 / rms passes through); without a weight the unit norm follows the rotation
    const float* nw = kind == 0 ? qnw : knw;         // (wave-uniform)
    if (nw != nullptr) {
#pragma unroll
      for (int e = 0; e < NE; ++e) {
        const int c = lane + 64 * e;
        s2 += v[e] * v[e];
        v[e] *= c < n ? nw[c] : 0.f;
      }
    }
#pragma unroll
    for (int e = 0; e < NE; ++e) {
      const int c = lane + 64 * e;
      const float other = __shfl_xor(v[e], 1, 64);
      if (c < rot) v[e] = (c & 1) ? v[e] * cs[e] + other * sn[e] : v[e] * cs[e] - other * sn[e];
      if (nw == nullptr) s2 += v[e] * v[e];           // (entries past n are zeros)
    }
    const float rs = 1.f / sqrtf(wave_sum(s2) / (float)n + eps);
    if (kind == 0) {
      float* qr = qo + (size_t)t * ldq + (size_t)hi * d;
#pragma unroll
      for (int e = 0; e < NE; ++e) { const int c = lane + 64 * e; if (c < n) qr[c] = v[e] * rs; }
    } else {
      TO* kr = kc + (size_t)kv_slot[t] * ldk + (size_t)(hi - H) * d;
#pragma unroll
      for (int e = 0; e < NE; ++e) { const int c = lane + 64 * e; if (c < n) stf(kr, c, v[e] * rs); }
    }
  }
}

template <typename TO>
static void qkv_launch(int TP, int ne, dim3 grid, hipStream_t st, const float* z, int ldz, const float* w, float* state, int taps,
                       const int* tok_seq, const int* tok_pos, const int* cu, const int* pos0, const int* slot, const int* kv_slot,
                       int H, int G, int d, int dv, float eps, const float* freqs, int rot, float* qo, int ldq, TO* kc, int ldk,
                       TO* vc, int ldv, int C, int fuse, int Gv, const float* qnw, const float* knw) {
#define QKV_GO(TT, NN) hipLaunchKernelGGL((qkv_conv_rope_kernel<TO, TT, NN>), grid, dim3(256), 0, st, z, ldz, w, state, taps, tok_seq, \
                                          tok_pos, cu, pos0, slot, kv_slot, H, G, d, dv, eps, freqs, rot, qo, ldq, kc, ldk, vc, ldv, C, fuse, \
                                          Gv, qnw, knw)
#define QKV_NE(TT) do { if (ne <= 1) QKV_GO(TT, 1); else if (ne <= 2) QKV_GO(TT, 2); else QKV_GO(TT, QKV_MAX_E); } while (0)
  if (TP == 2) QKV_NE(2);
  else if (TP == 3) QKV_NE(3);
  else if (TP == 4) QKV_NE(4);
  else QKV_NE(0);
#undef QKV_NE
#undef QKV_GO
}

extern "C" int fls_seq_qkv_conv_rope(const float* z, int ldz, const float* w, float* state, int taps, const int* tok_seq,
                                     const int* tok_pos, const int* cu, const int* pos0, const int* slot, const int* kv_slot,
                                     int T, int B, int H, int G, int d, int dv, float eps, const float* freqs, int rot, float* qo,
                                     int ldq, void* kc, int ldk, void* vc, int ldv, int tc, int one_row_each, int Gv,
                                     const float* qnw, const float* knw, fls_stream_t s) {
  if (T <= 0) return 0;
  if (Gv < 0 || G == 0) Gv = G;
  if (H < 1 || G < 0 || d < 1 || d > 64 * QKV_MAX_E || dv > 64 * QKV_MAX_E || rot < 0 || rot > d || (rot & 1) ||
      (rot > 0 && freqs == nullptr) || (G > 0 && (kc == nullptr || vc == nullptr || kv_slot == nullptr || dv < 1)) ||
      (w != nullptr && (taps < 1 || (taps > 1 && state == nullptr))))
    return -1;
  const int C = H * d + G * d + Gv * dv;
  if (C > ldz || H * d > ldq || (G > 0 && (G * d > ldk || Gv * dv > ldv))) return -1;
  const int ipr = H + G + Gv;
  // blocks per row: one when the rows alone fill the chip (every wave then reuses its sines and cosines for a
  // quarter of the row's heads), up to a wave per head when rows are few
  const int per_row_max = (ipr + 3) / 4;
  int per_row = (2048 + T - 1) / T;
  per_row = per_row < 1 ? 1 : (per_row > per_row_max ? per_row_max : per_row);
  const int fuse = one_row_each && T == B;
  dim3 grid(T, per_row);
  hipStream_t st = (hipStream_t)s;
  const int TP = (w != nullptr && taps >= 2 && taps <= 4) ? taps : 0;
  const int ne = ((d > dv ? d : dv) + 63) / 64;
  if (tc == 1) qkv_launch<bf16_t>(TP, ne, grid, st, z, ldz, w, state, taps, tok_seq, tok_pos, cu, pos0, slot, kv_slot, H, G, d, dv, eps, freqs, rot, qo, ldq, (bf16_t*)kc, ldk, (bf16_t*)vc, ldv, C, fuse, Gv, qnw, knw);
  else qkv_launch<float>(TP, ne, grid, st, z, ldz, w, state, taps, tok_seq, tok_pos, cu, pos0, slot, kv_slot, H, G, d, dv, eps, freqs, rot, qo, ldq, (float*)kc, ldk, (float*)vc, ldv, C, fuse, Gv, qnw, knw);
  SEQ_LAUNCH_CHECK();
  if (w != nullptr && taps > 1 && !fuse) {
    hipLaunchKernelGGL(conv_state_kernel, dim3((C + 255) / 256, B), dim3(256), 0, st, z, ldz, state, cu, pos0, slot, C, taps);
    SEQ_LAUNCH_CHECK();
  }
  return 0;
}

// ------------------------------------------------------------------- gated linear recurrence
// one thread per (request, channel); sqrt(1 - a^2) from expm1 of the log decay, which keeps its
// accuracy when a is close to 1
template <typename TO>
__global__ void rglru_scan_kernel(const float* __restrict__ u, int ldu, const float* __restrict__ g, int ldg,
                                  const float* __restrict__ lam, const float* __restrict__ y, int ldy, float* __restrict__ state,
                                  TO* __restrict__ out, int ldo, const int* __restrict__ cu, const int* __restrict__ pos0,
                                  const int* __restrict__ slot, int W, float cdecay) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= W) return;
  const int a0 = cu[s], a1 = cu[s + 1];
  float* sp = state + (size_t)slot[s] * W + c;
  float S = pos0[s] > 0 ? *sp : 0.f;
  const float k = -cdecay * softplus_f(lam[c]);
  for (int t0 = a0; t0 < a1; t0 += 4) {
    // the four rows' inputs first (independent of S), then the dependent chain
    float gr[4], gi[4], uv[4], yv[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int t = min(t0 + j, a1 - 1);
      gr[j] = g[(size_t)t * ldg + c];
      gi[j] = g[(size_t)t * ldg + W + c];
      uv[j] = u[(size_t)t * ldu + c];
      yv[j] = y[(size_t)t * ldy + c];
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (t0 + j < a1) {
        const float la = k * sigmoid_f(gr[j]);                  // log a_t <= 0
        S = expf(la) * S + sqrtf(-expm1f(2.f * la)) * sigmoid_f(gi[j]) * uv[j];
        stf(out + (size_t)(t0 + j) * ldo, c, S * gelu_tanh_f(yv[j]));
      }
    }
  }
  *sp = S;
}

extern "C" int fls_seq_rglru_scan(const float* u, int ldu, const float* g, int ldg, const float* lam, const float* y, int ldy,
                                  float* state, void* out, int to, int ldo, const int* cu, const int* pos0, const int* slot,
                                  int B, int W, float c, fls_stream_t s) {
  if (B <= 0) return 0;
  dim3 grid((W + 127) / 128, B);
  if (to == 1) hipLaunchKernelGGL((rglru_scan_kernel<bf16_t>), grid, dim3(128), 0, (hipStream_t)s, u, ldu, g, ldg, lam, y, ldy, state, (bf16_t*)out, ldo, cu, pos0, slot, W, c);
  else hipLaunchKernelGGL((rglru_scan_kernel<float>), grid, dim3(128), 0, (hipStream_t)s, u, ldu, g, ldg, lam, y, ldy, state, (float*)out, ldo, cu, pos0, slot, W, c);
  SEQ_LAUNCH_CHECK();
  return 0;
}

// The same recurrence for steps with many rows per request, in three passes over row tiles (each tile:
// up to 128 consecutive rows of one request; tile_cu[s] .. tile_cu[s + 1] are request s's tiles):
//   1. per (tile, channel): the tile's decay A = prod a_t and its state from zero L (S_out = A S_in + L);
//   2. per (request, channel): walk the request's tiles, leaving each tile's incoming state in place of L;
//   3. per (tile, channel): replay the tile from its incoming state and write the gated outputs.
// A thread of the plain kernel walks a whole prompt alone; here T / 128 times as many threads run.
__device__ __forceinline__ void rglru_ab(float gr, float gi, float uv, float k, float& a, float& b) {
  const float la = k * sigmoid_f(gr);
  a = expf(la);
  b = sqrtf(-expm1f(2.f * la)) * sigmoid_f(gi) * uv;
}

__global__ void rglru_tile_reduce_kernel(const float* __restrict__ u, int ldu, const float* __restrict__ g, int ldg,
                                         const float* __restrict__ lam, const int* __restrict__ tiles, float* __restrict__ TA,
                                         float* __restrict__ TL, int W, float cdecay) {
  const int tile = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= W) return;
  const int a0 = tiles[2 * tile], a1 = a0 + tiles[2 * tile + 1];
  const float k = -cdecay * softplus_f(lam[c]);
  float A = 1.f, L = 0.f;
  for (int t0 = a0; t0 < a1; t0 += 4) {
    float gr[4], gi[4], uv[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int t = min(t0 + j, a1 - 1);
      gr[j] = g[(size_t)t * ldg + c];
      gi[j] = g[(size_t)t * ldg + W + c];
      uv[j] = u[(size_t)t * ldu + c];
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (t0 + j < a1) {
        float a, b;
        rglru_ab(gr[j], gi[j], uv[j], k, a, b);
        L = a * L + b;
        A *= a;
      }
    }
  }
  TA[(size_t)tile * W + c] = A;
  TL[(size_t)tile * W + c] = L;
}

__global__ void rglru_tile_carry_kernel(const float* __restrict__ TA, float* __restrict__ TL, float* __restrict__ state,
                                        const int* __restrict__ tile_cu, const int* __restrict__ pos0,
                                        const int* __restrict__ slot, int W) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= W) return;
  float* sp = state + (size_t)slot[s] * W + c;
  float S = pos0[s] > 0 ? *sp : 0.f;
  for (int tile = tile_cu[s]; tile < tile_cu[s + 1]; ++tile) {
    const float L = TL[(size_t)tile * W + c];
    TL[(size_t)tile * W + c] = S;                       // the tile's incoming state
    S = TA[(size_t)tile * W + c] * S + L;
  }
  *sp = S;
}

template <typename TO>
__global__ void rglru_tile_apply_kernel(const float* __restrict__ u, int ldu, const float* __restrict__ g, int ldg,
                                        const float* __restrict__ lam, const float* __restrict__ y, int ldy,
                                        const int* __restrict__ tiles, const float* __restrict__ TS, TO* __restrict__ out,
                                        int ldo, int W, float cdecay) {
  const int tile = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= W) return;
  const int a0 = tiles[2 * tile], a1 = a0 + tiles[2 * tile + 1];
  const float k = -cdecay * softplus_f(lam[c]);
  float S = TS[(size_t)tile * W + c];
  for (int t0 = a0; t0 < a1; t0 += 4) {
    float gr[4], gi[4], uv[4], yv[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int t = min(t0 + j, a1 - 1);
      gr[j] = g[(size_t)t * ldg + c];
      gi[j] = g[(size_t)t * ldg + W + c];
      uv[j] = u[(size_t)t * ldu + c];
      yv[j] = y[(size_t)t * ldy + c];
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (t0 + j < a1) {
        float a, b;
        rglru_ab(gr[j], gi[j], uv[j], k, a, b);
        S = a * S + b;
        stf(out + (size_t)(t0 + j) * ldo, c, S * gelu_tanh_f(yv[j]));
      }
    }
  }
}

extern "C" int fls_seq_rglru_scan_tiled(const float* u, int ldu, const float* g, int ldg, const float* lam, const float* y,
                                        int ldy, float* state, void* out, int to, int ldo, const int* tiles, int n_tiles,
                                        const int* tile_cu, float* scratch, const int* pos0, const int* slot, int B, int W,
                                        float c, fls_stream_t s) {
  if (B <= 0 || n_tiles <= 0) return 0;
  hipStream_t st = (hipStream_t)s;
  float* TA = scratch;
  float* TL = scratch + (size_t)n_tiles * W;
  dim3 gt((W + 127) / 128, n_tiles), gb((W + 127) / 128, B);
  hipLaunchKernelGGL(rglru_tile_reduce_kernel, gt, dim3(128), 0, st, u, ldu, g, ldg, lam, tiles, TA, TL, W, c);
  SEQ_LAUNCH_CHECK();
  hipLaunchKernelGGL(rglru_tile_carry_kernel, gb, dim3(128), 0, st, TA, TL, state, tile_cu, pos0, slot, W);
  SEQ_LAUNCH_CHECK();
  if (to == 1) hipLaunchKernelGGL((rglru_tile_apply_kernel<bf16_t>), gt, dim3(128), 0, st, u, ldu, g, ldg, lam, y, ldy, tiles, TL, (bf16_t*)out, ldo, W, c);
  else hipLaunchKernelGGL((rglru_tile_apply_kernel<float>), gt, dim3(128), 0, st, u, ldu, g, ldg, lam, y, ldy, tiles, TL, (float*)out, ldo, W, c);
  SEQ_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- selective state-space scan
// A block serves (request, head, a tile of value columns p).  The N x P state of the head is cut
// over threads: NS consecutive lanes share one column p, each keeping <= 16 state rows n in
// registers (n = i * NS + ns, so the lanes of a column read consecutive LDS words).  The step's rows
// are walked 16 at a time: the block first stages B_t, C_t (N floats each), x_t and z_t of its
// columns and the two per-row scalars dt_t = softplus(dt + bias) and exp(-exp(A) dt_t) in LDS with
// coalesced loads, then every thread runs the 16 steps of the recurrence out of LDS:
// S = decay * S + dt * B[n] * x[p], y = sum_n S[n] * C[n], the partial sums of the NS lanes folded with
// lane shuffles.
#define SSD_NPT 16
#define SSD_TT 16
template <int NS>
__global__ __launch_bounds__(256) void ssd_scan_kernel(const float* __restrict__ xbc, int ldx, const float* __restrict__ z, int ldz,
                                                       const float* __restrict__ dt, int lddt, const float* __restrict__ dt_bias,
                                                       const float* __restrict__ A_log, const float* __restrict__ Dskip,
                                                       float* __restrict__ state, float* __restrict__ out, int ldo,
                                                       const int* __restrict__ cu, const int* __restrict__ pos0,
                                                       const int* __restrict__ slot, int nh, int P, int N, int G) {
  constexpr int PPB = 256 / NS;                    // value columns per block
  constexpr int NMAX = NS * SSD_NPT;               // state rows the lanes of a column cover
  __shared__ float Bs[SSD_TT][NMAX], Cs[SSD_TT][NMAX];
  __shared__ float xs[SSD_TT][PPB], zs[SSD_TT][PPB];
  __shared__ float dts[SSD_TT], decs[SSD_TT];
  const int s = blockIdx.z, h = blockIdx.y;
  const int ns = threadIdx.x % NS, pl = threadIdx.x / NS;
  const int p0 = blockIdx.x * PPB;
  const int p = p0 + pl;
  const bool live = p < P;
  const int grp = h / (nh / G);
  const int inner = nh * P;
  const int a0 = cu[s], a1 = cu[s + 1];
  float S[SSD_NPT];
  float* sp = state + (((size_t)slot[s] * nh + h) * N) * P + (live ? p : 0);
  const bool carried = pos0[s] > 0;
#pragma unroll
  for (int i = 0; i < SSD_NPT; ++i) {
    const int n = i * NS + ns;
    S[i] = (carried && live && n < N) ? sp[(size_t)n * P] : 0.f;
  }
  const float negA = -expf(A_log[h]), db = dt_bias[h], dsk = Dskip[h];
  for (int t0 = a0; t0 < a1; t0 += SSD_TT) {
    const int nt = min(SSD_TT, a1 - t0);
    __syncthreads();
    for (int e = threadIdx.x; e < nt * NMAX; e += 256) {
      const int tt = e / NMAX, n = e % NMAX;
      const float* row = xbc + (size_t)(t0 + tt) * ldx + inner + grp * N;
      Bs[tt][n] = n < N ? row[n] : 0.f;
      Cs[tt][n] = n < N ? row[G * N + n] : 0.f;
    }
    for (int e = threadIdx.x; e < nt * PPB; e += 256) {
      const int tt = e / PPB, c = e % PPB;
      const bool ok = p0 + c < P;
      xs[tt][c] = ok ? xbc[(size_t)(t0 + tt) * ldx + h * P + p0 + c] : 0.f;
      zs[tt][c] = ok ? z[(size_t)(t0 + tt) * ldz + h * P + p0 + c] : 0.f;
    }
    if ((int)threadIdx.x < nt) {
      const float dtv = softplus_f(dt[(size_t)(t0 + threadIdx.x) * lddt + h] + db);
      dts[threadIdx.x] = dtv;
      decs[threadIdx.x] = expf(negA * dtv);
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float dec = decs[tt], xv = xs[tt][pl];
      const float dx = dts[tt] * xv;
      float yv = 0.f;
#pragma unroll
      for (int i = 0; i < SSD_NPT; ++i) {
        const int n = i * NS + ns;
        S[i] = dec * S[i] + dx * Bs[tt][n];
        yv += S[i] * Cs[tt][n];
      }
#pragma unroll
      for (int o = NS / 2; o > 0; o >>= 1) yv += __shfl_xor(yv, o, 64);
      if (ns == 0 && live) out[(size_t)(t0 + tt) * ldo + h * P + p] = (yv + dsk * xv) * silu_f(zs[tt][pl]);
    }
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < SSD_NPT; ++i) {
      const int n = i * NS + ns;
      if (n < N) sp[(size_t)n * P] = S[i];
    }
  }
}

extern "C" int fls_seq_ssd_scan(const float* xbc, int ldx, const float* z, int ldz, const float* dt, int lddt,
                                const float* dt_bias, const float* A_log, const float* Dskip, float* state, float* out, int ldo,
                                const int* cu, const int* pos0, const int* slot, int B, int nh, int P, int N, int G,
                                fls_stream_t s) {
  if (B <= 0) return 0;
  if (N < 1 || N > 256 || G < 1 || nh % G) return -1;
  int nsl = 1;
  while (nsl * SSD_NPT < N) nsl *= 2;
  hipStream_t st = (hipStream_t)s;
#define SSD_LAUNCH(NSV) hipLaunchKernelGGL((ssd_scan_kernel<NSV>), dim3((P + 256 / NSV - 1) / (256 / NSV), nh, B), dim3(256), 0, st, \
    xbc, ldx, z, ldz, dt, lddt, dt_bias, A_log, Dskip, state, out, ldo, cu, pos0, slot, nh, P, N, G)
  switch (nsl) {
    case 1: SSD_LAUNCH(1); break;
    case 2: SSD_LAUNCH(2); break;
    case 4: SSD_LAUNCH(4); break;
    case 8: SSD_LAUNCH(8); break;
    default: SSD_LAUNCH(16); break;
  }
#undef SSD_LAUNCH
  SEQ_LAUNCH_CHECK();
  return 0;
}
