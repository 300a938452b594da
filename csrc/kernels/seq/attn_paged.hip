// Attention of packed rows over paged keys and values, for prompts and for decoding alike: softmax
// over the visible keys, or (gate_bias given) every key weighted by sigmoid(score + gate_bias[h]) on its
// own.  Visible: j <= i inside the row's chunk and / or window, plus, with keep_first, the first
// keep_first keys of the sequence however far back they lie.  Keys and values are the first G d and
// G dv columns of pool rows ldk and ldv wide, so both may be one pool (values = a prefix of the keys:
// attention over latent rows).  The query may be fp32 while the pools hold bf16.  has_sink: the softmax
// has one more entry of score `sink` and no value (p_j = exp(s_j) / (exp(sink) + sum exp(s))); head_gate
// [T, H] fp32: the output of (row, head) times sigmoid(head_gate[t, h]).
//
// One block (four wavefronts) per (row, query head).  The row's query sits in LDS as fp32.  The keys
// it may see -- j <= i, inside its chunk of the sequence and / or its window -- are walked in tiles of
// 64, the four waves taking tiles in turn:
//   scores : lane = key.  The lane finds its key's row in the request's page table, reads the key
//            (16-byte loads when the head size allows) against the query in LDS, scales, caps
//            (cap * tanh(s / cap)) and subtracts the distance penalty r1 * log(1 + r2 * (i - j));
//   softmax: running maximum and sum per wave (online), weights to LDS;
//   values : lane = value column.  Every lane walks the tile's keys, reading the value rows
//            coalesced, and accumulates its columns in registers (up to 8 x 64 columns).
// The four waves' (maximum, sum, accumulator) are merged through LDS at the end.  All of it is fp32;
// only the stored keys / values and the output have the model's element type.  A decoded token is
// one row, so its block walks the (bounded) chunk or window with four waves; a prompt has one block
// per row and head, which fills the chip without a second kernel.
#include "seq_common.h"
#include "fls_seq.h"

#define MAX_DV_PER_LANE 8      // value columns per lane: head value size <= 512 (a latent row)
#define MAX_D 1024

template <typename T>
__device__ __forceinline__ float dot_row(const T* __restrict__ k, const float* __restrict__ q, int d, int vec) {
  float acc = 0.f;
  if (vec) {
    if constexpr (sizeof(T) == 2) {
      for (int c = 0; c < d; c += 8) {
        const uint4 v = *reinterpret_cast<const uint4*>(k + c);
        const bf16_t* e = reinterpret_cast<const bf16_t*>(&v);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc += bf16_to_f(e[i]) * q[c + i];
      }
    } else {
      for (int c = 0; c < d; c += 4) {
        const float4 v = *reinterpret_cast<const float4*>(k + c);
        acc += v.x * q[c] + v.y * q[c + 1] + v.z * q[c + 2] + v.w * q[c + 3];
      }
    }
  } else {
    for (int c = 0; c < d; ++c) acc += ldf(k, c) * q[c];
  }
  return acc;
}

template <typename TQ, typename T, typename TO>
__global__ __launch_bounds__(256) void attn_paged_kernel(const TQ* __restrict__ q, int ldq, const T* kc, int ldk,
                                                         const T* vc, int ldv, TO* __restrict__ out, int ldo,
                                                         const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
                                                         const int* __restrict__ page_table, int pt_stride, int H, int G,
                                                         int d, int dv, float scale, float softcap,
                                                         const float* __restrict__ r1, const float* __restrict__ r2,
                                                         int chunk, int window, int keep_first,
                                                         const float* __restrict__ gate_bias, float out_scale,
                                                         int page_size, int vec, float* __restrict__ part, int has_sink,
                                                         float sink, const float* __restrict__ head_gate, int ldhg, int Gv) {
  __shared__ float qs[MAX_D];
  __shared__ float pw[4][64];
  __shared__ int prow[4][64];
  __shared__ float mm[4], ll[4];
  __shared__ float accs[4][MAX_DV_PER_LANE * 64];
  const int t = blockIdx.y, h = blockIdx.x;
  const int g = h / (H / G);
  const int gv = g % Gv;                          // (several score maps over the same values: Gv < G value heads)
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int i = tok_pos[t];
  const int* table = page_table + (size_t)tok_seq[t] * pt_stride;
  for (int c = threadIdx.x; c < d; c += 256) qs[c] = ldf(q + (size_t)t * ldq + (size_t)h * d, c);
  __syncthreads();
  int lo = chunk > 0 ? (i / chunk) * chunk : 0;
  if (window > 0 && i - window + 1 > lo) lo = i - window + 1;
  const int nkeep = min(keep_first, lo);          // kept first keys that the window no longer covers
  const int nkeys = nkeep + i - lo + 1;
  const int ntiles = (nkeys + 63) / 64;
  const float a1 = r1 != nullptr ? r1[h] : 0.f, a2 = r2 != nullptr ? r2[h] : 0.f;
  const bool gated = gate_bias != nullptr;
  const float gb = gated ? gate_bias[h] : 0.f;
  float m = -1e30f, l = 0.f;
  float acc[MAX_DV_PER_LANE];
#pragma unroll
  for (int c = 0; c < MAX_DV_PER_LANE; ++c) acc[c] = 0.f;
  // gridDim.z > 1: the key tiles are cut into gridDim.z ranges, one block each, whose (maximum, sum,
  // weighted values) go to `part` and are merged by attn_merge_kernel
  const int nsplit = gridDim.z;
  const int tps = (ntiles + nsplit - 1) / nsplit;
  const int tile_hi = min(ntiles, ((int)blockIdx.z + 1) * tps);
  for (int tile = blockIdx.z * tps + wave; tile < tile_hi; tile += 4) {
    const int n = tile * 64 + lane;
    const bool valid = n < nkeys;
    const int j = n < nkeep ? n : lo + (n - nkeep);
    float sc = -1e30f;
    int row = 0;
    if (valid) {
      row = table[j / page_size] * page_size + j % page_size;
      sc = dot_row<T>(kc + (size_t)row * ldk + (size_t)g * d, qs, d, vec) * scale;
      if (softcap > 0.f) sc = softcap * tanhf(sc / softcap);
      if (a1 != 0.f) sc -= a1 * log1pf(a2 * (float)(i - j));
    }
    float p, corr = 1.f;
    if (gated) {
      p = valid ? sigmoid_f(sc + gb) : 0.f;
    } else {
      const float mt = fmaxf(m, wave_max(sc));
      p = valid ? expf(sc - mt) : 0.f;
      corr = expf(m - mt);
      l = l * corr + wave_sum(p);
      m = mt;
    }
    pw[wave][lane] = p;
    prow[wave][lane] = row;
    // (a wave reads back only what its own lanes wrote: LDS ordering within a wave needs no barrier,
    // but the compiler must not move the loads above the stores)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    const int nk = min(64, nkeys - tile * 64);
#pragma unroll
    for (int c = 0; c < MAX_DV_PER_LANE; ++c) {
      const int e = lane + 64 * c;
      if (e < dv) {
        float a = acc[c] * corr;
        int jj = 0;
        for (; jj + 8 <= nk; jj += 8) {            // eight independent value loads in flight
          float v[8];
#pragma unroll
          for (int x = 0; x < 8; ++x) v[x] = ldf(vc + (size_t)prow[wave][jj + x] * ldv + (size_t)gv * dv, e);
#pragma unroll
          for (int x = 0; x < 8; ++x) a += pw[wave][jj + x] * v[x];
        }
        for (; jj < nk; ++jj) a += pw[wave][jj] * ldf(vc + (size_t)prow[wave][jj] * ldv + (size_t)gv * dv, e);
        acc[c] = a;
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  if (lane == 0) { mm[wave] = m; ll[wave] = l; }
#pragma unroll
  for (int c = 0; c < MAX_DV_PER_LANE; ++c) accs[wave][lane + 64 * c] = acc[c];
  __syncthreads();
  if (wave == 0) {
    float f[4], inv = out_scale, mx = 0.f, lt = 0.f;
    if (gated) {
#pragma unroll
      for (int w = 0; w < 4; ++w) f[w] = 1.f;
    } else {
      mx = fmaxf(fmaxf(mm[0], mm[1]), fmaxf(mm[2], mm[3]));
      if (has_sink && nsplit == 1) mx = fmaxf(mx, sink);          // (with ranges the merge adds the silent entry, once)
#pragma unroll
      for (int w = 0; w < 4; ++w) { f[w] = expf(mm[w] - mx); lt += ll[w] * f[w]; }
      if (has_sink && nsplit == 1) lt += expf(sink - mx);
      inv = out_scale / lt;
    }
    if (head_gate != nullptr) inv *= sigmoid_f(head_gate[(size_t)t * ldhg + h]);
    if (nsplit > 1) {                              // this range's share, not yet normalised
      float* pp = part + (((size_t)t * H + h) * nsplit + blockIdx.z) * (dv + 4);      // record: values[dv] | maximum | sum | pad
      if (lane == 0) { pp[dv] = mx; pp[dv + 1] = lt; }
#pragma unroll
      for (int c = 0; c < MAX_DV_PER_LANE; ++c) {
        const int e = lane + 64 * c;
        if (e < dv) pp[e] = accs[0][e] * f[0] + accs[1][e] * f[1] + accs[2][e] * f[2] + accs[3][e] * f[3];
      }
      return;
    }
#pragma unroll
    for (int c = 0; c < MAX_DV_PER_LANE; ++c) {
      const int e = lane + 64 * c;
      if (e < dv) {
        const float v = accs[0][e] * f[0] + accs[1][e] * f[1] + accs[2][e] * f[2] + accs[3][e] * f[3];
        stf(out + (size_t)t * ldo + (size_t)h * dv, e, v * inv);
      }
    }
  }
}

// out[t, h] from the nsplit partial results of a (row, head): softmax parts are rescaled to the common
// maximum and divided by the total sum, gated parts are added.  The nsplit weights are worked out once
// per block (nsplit <= MERGE_MAX_SPLIT), then every thread sums its value columns over the parts.
#define MERGE_MAX_SPLIT 64
template <typename T>
__global__ void attn_merge_kernel(const float* __restrict__ part, T* __restrict__ out, int ldo, int H, int dv, int nsplit, int gated,
                                  float out_scale, int has_sink, float sink, const float* __restrict__ head_gate, int ldhg) {
  __shared__ float wz[MERGE_MAX_SPLIT];
  const int t = blockIdx.y, h = blockIdx.x;
  const int rs = dv + 4;                           // record: values[dv] | maximum | sum | pad
  const float* pp = part + ((size_t)t * H + h) * nsplit * rs;
  if (threadIdx.x < 64) {                          // (one wave: lane z holds part z's maximum and sum)
    const int z = threadIdx.x;
    const float mz = (z < nsplit && !gated) ? pp[z * rs + dv] : -1e30f;
    const float lz = (z < nsplit && !gated) ? pp[z * rs + dv + 1] : 0.f;
    float mx = wave_max(mz);
    if (has_sink) mx = fmaxf(mx, sink);
    const float f = expf(mz - mx);
    float lt = wave_sum(lz * f);
    if (has_sink) lt += expf(sink - mx);
    const float os = head_gate != nullptr ? out_scale * sigmoid_f(head_gate[(size_t)t * ldhg + h]) : out_scale;
    wz[z] = gated ? os : f * os / lt;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < dv; e += blockDim.x) {
    float v = 0.f;
    for (int z = 0; z < nsplit; ++z) v += pp[z * rs + e] * wz[z];
    stf(out + (size_t)t * ldo + (size_t)h * dv, e, v);
  }
}

// (also used by the matrix-core kernels that cut a row's keys over blocks)
int seq_attn_merge(const float* part, void* out, int tc, int ldo, int T, int H, int dv, int nsplit, int gated, float out_scale,
                   int has_sink, float sink, const float* head_gate, int ldhg, fls_stream_t s) {
  const int threads = dv > 128 ? 256 : (dv > 64 ? 128 : 64);
  hipStream_t st = (hipStream_t)s;
  if (tc == 1) hipLaunchKernelGGL((attn_merge_kernel<bf16_t>), dim3(H, T), dim3(threads), 0, st, part, (bf16_t*)out, ldo, H, dv, nsplit, gated, out_scale, has_sink, sink, head_gate, ldhg);
  else hipLaunchKernelGGL((attn_merge_kernel<float>), dim3(H, T), dim3(threads), 0, st, part, (float*)out, ldo, H, dv, nsplit, gated, out_scale, has_sink, sink, head_gate, ldhg);
  SEQ_LAUNCH_CHECK();
  return 0;
}

// tq: type of q; tc: type of the pools; to: type of out (fp32 over bf16 pools allowed)
extern "C" int fls_seq_attn_paged(const void* q, int ldq, int tq, const void* kc, int ldk, const void* vc, int ldv, int tc,
                                  void* out, int to, int ldo, const int* tok_seq, const int* tok_pos, const int* page_table,
                                  int pt_stride, int T, int H, int G, int d, int dv, float scale, float softcap,
                                  const float* r1, const float* r2, int chunk, int window, int keep_first,
                                  const float* gate_bias, float out_scale, int page_size, int nsplit, float* part,
                                  int has_sink, float sink, const float* head_gate, int ldhg, int Gv, fls_stream_t s) {
  if (T <= 0) return 0;
  if (Gv <= 0) Gv = G;
  if (G % Gv || (to == 1 && tc == 0)) return -1;
  if (has_sink && gate_bias != nullptr) return -1;      // (a silent entry belongs to a softmax)
  if (nsplit < 1 || nsplit > MERGE_MAX_SPLIT || (nsplit > 1 && part == nullptr)) return -1;
  if (d > MAX_D || dv > 64 * MAX_DV_PER_LANE || G < 1 || H % G || page_size < 1 || G * d > ldk || Gv * dv > ldv || keep_first < 0
      || (tq == 1 && tc == 0)) return -1;
  dim3 grid(H, T, nsplit);
  hipStream_t st = (hipStream_t)s;
#define ATTN_PAGED_ARGS ldq, (const TC*)kc, ldk, (const TC*)vc, ldv, (TOUT*)out, ldo, tok_seq, tok_pos, page_table, pt_stride, H, G, \
                        d, dv, scale, softcap, r1, r2, chunk, window, keep_first, gate_bias, out_scale, page_size, vec, part, has_sink, sink, \
                        nsplit > 1 ? nullptr : head_gate, ldhg, Gv
  if (tc == 1) {
    using TC = bf16_t;
    const int vec = d % 8 == 0 && (uintptr_t)kc % 16 == 0 && ldk % 8 == 0;
    if (to == 0) {
      using TOUT = float;
      if (tq == 1) hipLaunchKernelGGL((attn_paged_kernel<bf16_t, bf16_t, float>), grid, dim3(256), 0, st, (const bf16_t*)q, ATTN_PAGED_ARGS);
      else hipLaunchKernelGGL((attn_paged_kernel<float, bf16_t, float>), grid, dim3(256), 0, st, (const float*)q, ATTN_PAGED_ARGS);
    } else {
      using TOUT = bf16_t;
      if (tq == 1) hipLaunchKernelGGL((attn_paged_kernel<bf16_t, bf16_t, bf16_t>), grid, dim3(256), 0, st, (const bf16_t*)q, ATTN_PAGED_ARGS);
      else hipLaunchKernelGGL((attn_paged_kernel<float, bf16_t, bf16_t>), grid, dim3(256), 0, st, (const float*)q, ATTN_PAGED_ARGS);
    }
  } else {
    using TC = float;
    using TOUT = float;
    const int vec = d % 4 == 0 && (uintptr_t)kc % 16 == 0 && ldk % 4 == 0;
    hipLaunchKernelGGL((attn_paged_kernel<float, float, float>), grid, dim3(256), 0, st, (const float*)q, ATTN_PAGED_ARGS);
  }
#undef ATTN_PAGED_ARGS
  SEQ_LAUNCH_CHECK();
  if (nsplit > 1) return seq_attn_merge(part, out, to, ldo, T, H, dv, nsplit, gate_bias != nullptr, out_scale, has_sink, sink, head_gate, ldhg, s);
  return 0;
}
