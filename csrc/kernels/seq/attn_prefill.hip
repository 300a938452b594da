// Prompt attention on the matrix cores, for bf16 models: the same masks (chunk, window, kept first
// keys), score cap, distance penalty and weights (softmax, or a sigmoid gate per key) as
// attn_paged_kernel, for steps that bring many rows per request.  Queries may come as fp32 (rounded to
// bf16 on their way into the fragments).  Keys of a row tile: first the kept first keys that lie before
// the tile's window (if any), then the window's keys, both walked 32 at a time.
//
// The host cuts every request's rows of the step into tiles of up to 128 consecutive rows; a block
// serves one tile and one query head, its four waves 32 query rows each.  Keys are walked 32 at a
// time, from the first key the tile's first row may see to the tile's last row, gathered from the
// request's pages into LDS: K as [key][d], V transposed as [column][key].  Per key tile and wave:
//   S^T = K Q^T        one 32x32x16 MFMA per 16 of d (Q fragments stay in registers): a lane then
//                      holds 16 keys' scores of ONE query (column = lane % 32), its partner lane ^ 32
//                      the other 16, so the softmax statistics are per-lane scalars: one shuffle
//                      per reduction, and the running maximum, sum and rescale factor live in the
//                      lane that owns the query;
//   scores             scale, cap, distance penalty, mask (chunk / window / causal) in fp32;
//   weights            exp in fp32, written to LDS as two bf16 terms (p = hi + lo, 16 mantissa bits
//                      together), so the value product loses nothing to a bf16 rounding of p;
//   O^T += V^T P^T     MFMAs again; O^T has the same column = query layout, so the rescale is a
//                      per-lane multiply.
#include "seq_common.h"
#include "fls_seq.h"

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

#define KT 32             // keys per tile
#define PLD (KT + 8)      // row stride (elements) of the transposed V tile and of the weight tiles

template <int D, int DV, typename TQ, typename TO>
__global__ __launch_bounds__(256) void attn_prefill_kernel(const TQ* __restrict__ q, int ldq, const bf16_t* __restrict__ kc, int ldk,
                                                           const bf16_t* __restrict__ vc, int ldv, TO* __restrict__ out, int ldo,
                                                           const int* __restrict__ tiles, const int* __restrict__ tok_seq,
                                                           const int* __restrict__ tok_pos, const int* __restrict__ page_table,
                                                           int pt_stride, int H, int G, float scale, float softcap,
                                                           const float* __restrict__ r1, const float* __restrict__ r2,
                                                           int chunk, int window, int keep_first,
                                                           const float* __restrict__ gate_bias, float out_scale, int page_size,
                                                           int has_sink, float sink, const float* __restrict__ head_gate,
                                                           int ldhg, int Gv) {
  constexpr int KLD = D + 8;
  __shared__ __attribute__((aligned(16))) bf16_t Ks[KT * KLD];
  __shared__ __attribute__((aligned(16))) bf16_t Vt[DV * PLD];
  __shared__ __attribute__((aligned(16))) bf16_t Ps[4][2][32 * PLD];
  const int h = blockIdx.x, g = h / (H / G);
  const int row0 = tiles[2 * blockIdx.y], nrows = tiles[2 * blockIdx.y + 1];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int ql = lane & 31, h2 = lane >> 5;
  const int* table = page_table + (size_t)tok_seq[row0] * pt_stride;
  const int i_first = tok_pos[row0], i_last = i_first + nrows - 1;
  // this lane's query
  const int qrow = wave * 32 + ql;
  const bool qok = qrow < nrows;
  const int iq = i_first + qrow;
  int lo_q = chunk > 0 ? (iq / chunk) * chunk : 0;
  if (window > 0 && iq - window + 1 > lo_q) lo_q = iq - window + 1;
  int lo_blk = chunk > 0 ? (i_first / chunk) * chunk : 0;
  if (window > 0 && i_first - window + 1 > lo_blk) lo_blk = i_first - window + 1;
  // the wave's rows span positions [w_first, w_last]; it skips key tiles none of them sees
  const int w_first = i_first + wave * 32, w_last = min(i_last, w_first + 31);
  int lo_w = chunk > 0 ? (w_first / chunk) * chunk : 0;
  if (window > 0 && w_first - window + 1 > lo_w) lo_w = w_first - window + 1;
  bf16x8 Qf[D / 16];
  {
    const TQ* qp = q + (size_t)(row0 + (qok ? qrow : 0)) * ldq + (size_t)h * D + h2 * 8;
#pragma unroll
    for (int s = 0; s < D / 16; ++s) {
      uint4 v = make_uint4(0, 0, 0, 0);
      if (qok) {
        if constexpr (sizeof(TQ) == 2) {
          v = *reinterpret_cast<const uint4*>(qp + 16 * s);
        } else {
          const float4 f0 = *reinterpret_cast<const float4*>(qp + 16 * s), f1 = *reinterpret_cast<const float4*>(qp + 16 * s + 4);
          bf16_t e[8] = {f_to_bf16(f0.x), f_to_bf16(f0.y), f_to_bf16(f0.z), f_to_bf16(f0.w),
                         f_to_bf16(f1.x), f_to_bf16(f1.y), f_to_bf16(f1.z), f_to_bf16(f1.w)};
          v = *reinterpret_cast<const uint4*>(e);
        }
      }
      Qf[s] = *reinterpret_cast<bf16x8*>(&v);
    }
  }
  floatx16 O[DV / 32];
#pragma unroll
  for (int c = 0; c < DV / 32; ++c)
#pragma unroll
    for (int r = 0; r < 16; ++r) O[c][r] = 0.f;
  // (the softmax's silent entry of score `sink`, if any, is where every query's running maximum and sum start)
  float m = has_sink ? sink : -1e30f, l = has_sink ? 1.f : 0.f;
  const float a1 = r1 != nullptr ? r1[h] : 0.f, a2 = r2 != nullptr ? r2[h] : 0.f;
  const bool gated = gate_bias != nullptr;
  const float gb = gated ? gate_bias[h] : 0.f;
  const float inv_cap = softcap > 0.f ? 1.f / softcap : 0.f;
  // key tiles: nt_keep tiles over the kept first keys [0, nkeep) that lie before the block's window,
  // then the tiles from lo_blk to the block's last row
  const int nkeep = min(keep_first, lo_blk);
  const int nt_keep = (nkeep + KT - 1) / KT;
  const int nt = nt_keep + (i_last - lo_blk) / KT + 1;
  // K / V of a key tile travel global -> registers -> LDS; the next tile's loads are issued before this
  // tile's matrix work and land in LDS after it, so the page gather's latency hides under the MFMAs
  constexpr int NK = KT * (D / 8) / 256, NV = KT * (DV / 8) / 256;
  static_assert(NK >= 1 && NV >= 1, "a tile has at least one 16-byte piece per thread");
  uint4 kreg[NK], vreg[NV];
  auto fetch = [&](int ti) {
    const int j0 = ti < nt_keep ? ti * KT : lo_blk + (ti - nt_keep) * KT;
    const int jend = ti < nt_keep ? nkeep : i_last + 1;
#pragma unroll
    for (int x = 0; x < NK; ++x) {
      const int e = threadIdx.x + 256 * x;
      const int kk = e / (D / 8), seg = e % (D / 8);
      const int j = j0 + kk;
      kreg[x] = make_uint4(0, 0, 0, 0);
      if (j < jend) {
        const size_t row = (size_t)table[j / page_size] * page_size + j % page_size;
        kreg[x] = *reinterpret_cast<const uint4*>(kc + row * ldk + (size_t)g * D + seg * 8);
      }
    }
#pragma unroll
    for (int x = 0; x < NV; ++x) {
      const int e = threadIdx.x + 256 * x;
      const int kk = e % KT, seg = e / KT;
      const int j = j0 + kk;
      vreg[x] = make_uint4(0, 0, 0, 0);
      if (j < jend) {
        const size_t row = (size_t)table[j / page_size] * page_size + j % page_size;
        vreg[x] = *reinterpret_cast<const uint4*>(vc + row * ldv + (size_t)(g % Gv) * DV + seg * 8);
      }
    }
  };
  fetch(0);
  for (int ti = 0; ti < nt; ++ti) {
    const bool kept = ti < nt_keep;
    const int j0 = kept ? ti * KT : lo_blk + (ti - nt_keep) * KT;
    const int jend = kept ? nkeep : i_last + 1;      // keys from jend on are padding of this tile
    __syncthreads();                          // the previous tile's readers are done
#pragma unroll
    for (int x = 0; x < NK; ++x) {
      const int e = threadIdx.x + 256 * x;
      *reinterpret_cast<uint4*>(Ks + (e / (D / 8)) * KLD + (e % (D / 8)) * 8) = kreg[x];
    }
#pragma unroll
    for (int x = 0; x < NV; ++x) {
      const int e = threadIdx.x + 256 * x;
      const int kk = e % KT, seg = e / KT;
      const bf16_t* ev = reinterpret_cast<const bf16_t*>(&vreg[x]);
#pragma unroll
      for (int y = 0; y < 8; ++y) Vt[(seg * 8 + y) * PLD + kk] = ev[y];
    }
    __syncthreads();
    if (ti + 1 < nt) fetch(ti + 1);
    if (wave * 32 >= nrows || (!kept && (j0 > w_last || (j0 + KT - 1 < lo_w && j0 >= keep_first)))) continue;   // (wave-uniform)
    floatx16 S;
#pragma unroll
    for (int r = 0; r < 16; ++r) S[r] = 0.f;
#pragma unroll
    for (int s = 0; s < D / 16; ++s) {
      const bf16x8 kf = *reinterpret_cast<const bf16x8*>(Ks + ql * KLD + 16 * s + h2 * 8);
      S = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, Qf[s], S, 0, 0, 0);
    }
    float p[16];
    float mt = -1e30f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int j = j0 + 8 * (r >> 2) + 4 * h2 + (r & 3);
      // (this kernel serves bf16 models only: the hardware exp / log are far inside their rounding)
      float sc = S[r] * scale;
      if (softcap > 0.f) sc = softcap * (1.f - 2.f / (__expf(2.f * sc * inv_cap) + 1.f));
      if (a1 != 0.f) sc -= a1 * __logf(1.f + a2 * (float)max(iq - j, 0));
      const bool vis = qok && j < jend && j <= iq && (j >= lo_q || j < keep_first);
      if (gated) p[r] = vis ? 1.f / (1.f + __expf(-(sc + gb))) : 0.f;
      else p[r] = vis ? sc : -1e30f;
      mt = fmaxf(mt, p[r]);
    }
    if (!gated) {
      mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
      mt = fmaxf(mt, m);
      float ps = 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        p[r] = p[r] > -1e29f ? __expf(p[r] - mt) : 0.f;
        ps += p[r];
      }
      ps += __shfl_xor(ps, 32, 64);
      const float corr = __expf(m - mt);
      l = l * corr + ps;
      m = mt;
#pragma unroll
      for (int c = 0; c < DV / 32; ++c)
#pragma unroll
        for (int r = 0; r < 16; ++r) O[c][r] *= corr;
    }
    bf16_t* ph = Ps[wave][0] + ql * PLD;
    bf16_t* pl = Ps[wave][1] + ql * PLD;
#pragma unroll
    for (int rg = 0; rg < 4; ++rg) {
      bf16_t hi[4], lo[4];
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        hi[x] = f_to_bf16(p[4 * rg + x]);
        lo[x] = f_to_bf16(p[4 * rg + x] - bf16_to_f(hi[x]));
      }
      *reinterpret_cast<uint2*>(ph + 8 * rg + 4 * h2) = *reinterpret_cast<const uint2*>(hi);
      *reinterpret_cast<uint2*>(pl + 8 * rg + 4 * h2) = *reinterpret_cast<const uint2*>(lo);
    }
    __builtin_amdgcn_wave_barrier();          // (a wave reads back its own lanes' writes: LDS is in order per wave)
#pragma unroll
    for (int ks = 0; ks < KT / 16; ++ks) {
      const bf16x8 bh = *reinterpret_cast<const bf16x8*>(ph + 16 * ks + 8 * h2);
      const bf16x8 bl = *reinterpret_cast<const bf16x8*>(pl + 16 * ks + 8 * h2);
#pragma unroll
      for (int c = 0; c < DV / 32; ++c) {
        const bf16x8 vf = *reinterpret_cast<const bf16x8*>(Vt + (32 * c + ql) * PLD + 16 * ks + 8 * h2);
        O[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, bh, O[c], 0, 0, 0);
        O[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, bl, O[c], 0, 0, 0);
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  if (qok && (gated || l > 0.f)) {
    float inv = gated ? out_scale : out_scale / l;
    if (head_gate != nullptr) inv *= sigmoid_f(head_gate[(size_t)(row0 + qrow) * ldhg + h]);
    TO* op = out + (size_t)(row0 + qrow) * ldo + (size_t)h * DV;
#pragma unroll
    for (int c = 0; c < DV / 32; ++c)
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        if constexpr (sizeof(TO) == 4) {
          *reinterpret_cast<float4*>(op + 32 * c + 8 * rg + 4 * h2) =
              make_float4(O[c][4 * rg] * inv, O[c][4 * rg + 1] * inv, O[c][4 * rg + 2] * inv, O[c][4 * rg + 3] * inv);
        } else {
          bf16_t o4[4];
#pragma unroll
          for (int x = 0; x < 4; ++x) o4[x] = f_to_bf16(O[c][4 * rg + x] * inv);
          *reinterpret_cast<uint2*>(op + 32 * c + 8 * rg + 4 * h2) = *reinterpret_cast<const uint2*>(o4);
        }
      }
  }
}

// tiles: n_tiles x (first packed row, rows <= 128) of one request each.  tq: type of q (0 fp32, 1 bf16);
// pools are bf16, out of type to.  Gv (0: G): value heads in the pool, key head g reads value head g % Gv.  Returns -2 for head sizes or alignments this kernel does not serve (the
// caller then runs fls_seq_attn_paged).
extern "C" int fls_seq_attn_prefill(const void* q, int ldq, int tq, const void* kc, int ldk, const void* vc, int ldv, void* out,
                                    int to, int ldo, const int* tiles, int n_tiles, const int* tok_seq, const int* tok_pos,
                                    const int* page_table, int pt_stride, int H, int G, int d, int dv, float scale,
                                    float softcap, const float* r1, const float* r2, int chunk, int window, int keep_first,
                                    const float* gate_bias, float out_scale, int page_size, int has_sink, float sink,
                                    const float* head_gate, int ldhg, int Gv, fls_stream_t s) {
  if (n_tiles <= 0) return 0;
  if (has_sink && gate_bias != nullptr) return -1;
  if (Gv <= 0) Gv = G;
  if (G < 1 || H % G || G % Gv || page_size < 1 || ldq % 8 || ldo % 4 || ldk % 8 || ldv % 8 || G * d > ldk || Gv * dv > ldv ||
      (uintptr_t)q % 16 || (uintptr_t)kc % 16 || (uintptr_t)vc % 16 || (uintptr_t)out % 16 || keep_first < 0)
    return -2;
  dim3 grid(H, n_tiles);
  hipStream_t st = (hipStream_t)s;
#define ATTN_PF_(DD, DDV, TQ_, TO_)                                                                                       \
  hipLaunchKernelGGL((attn_prefill_kernel<DD, DDV, TQ_, TO_>), grid, dim3(256), 0, st, (const TQ_*)q, ldq,                \
                     (const bf16_t*)kc, ldk, (const bf16_t*)vc, ldv, (TO_*)out, ldo, tiles, tok_seq, tok_pos,             \
                     page_table, pt_stride, H, G, scale, softcap, r1, r2, chunk, window, keep_first, gate_bias,           \
                     out_scale, page_size, has_sink, sink, head_gate, ldhg, Gv)
#define ATTN_PF(DD, DDV)                                                                                                  \
  do {                                                                                                                    \
    if (tq == 1 && to == 1) ATTN_PF_(DD, DDV, bf16_t, bf16_t);                                                            \
    else if (tq == 1) ATTN_PF_(DD, DDV, bf16_t, float);                                                                   \
    else if (to == 1) ATTN_PF_(DD, DDV, float, bf16_t);                                                                   \
    else ATTN_PF_(DD, DDV, float, float);                                                                                 \
  } while (0)
  if (d == 128 && dv == 128) ATTN_PF(128, 128);
  else if (d == 64 && dv == 64) ATTN_PF(64, 64);
  else if (d == 128 && dv == 64) ATTN_PF(128, 64);
  else if (d == 64 && dv == 128) ATTN_PF(64, 128);
  else return -2;
#undef ATTN_PF
#undef ATTN_PF_
  SEQ_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- few rows, many heads on one key/value head
// Decode rows of an attention whose query heads share one key / value head -- attention over cached latent
// rows: every head reads the same long rows (keys D wide, values their first DV columns or a pool of their
// own).  Here the HEADS of one token are the 32 query columns of the MFMA tile: a block serves (token,
// key/value head, range of key tiles), stages each tile of 32 rows once in LDS for all heads, and its four
// waves share the score product's operands but own a quarter of the value columns each, so every wave
// keeps DV / 4 accumulator columns.  All waves compute the same scores and softmax statistics (no exchange
// between them); the weights go to LDS as bf16 pairs as above.  A block whose range is one of several
// leaves (maximum, sum, weighted values) in `part` for attn_merge_kernel.
template <int D, int DV>
__global__ __launch_bounds__(256) void attn_heads_kernel(const float* __restrict__ q, int ldq, const bf16_t* kc, int ldk,
                                                         const bf16_t* vc, int ldv, bf16_t* __restrict__ out, int ldo,
                                                         const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
                                                         const int* __restrict__ page_table, int pt_stride, int H, int G,
                                                         float scale, int window, int keep_first, float out_scale,
                                                         int page_size, float* __restrict__ part) {
  constexpr int KLD = D + 8;
  constexpr int CPW = DV / 128;               // 32-column blocks of the values per wave
  __shared__ __attribute__((aligned(16))) bf16_t Ks[KT * KLD];
  __shared__ __attribute__((aligned(16))) bf16_t Vt[DV * PLD];
  __shared__ __attribute__((aligned(16))) bf16_t Ps[4][2][32 * PLD];
  const int t = blockIdx.x, g = blockIdx.y, nsplit = gridDim.z;
  const int nh = H / G;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int ql = lane & 31, h2 = lane >> 5;
  const int* table = page_table + (size_t)tok_seq[t] * pt_stride;
  const int i = tok_pos[t];
  const int lo = window > 0 ? max(0, i - window + 1) : 0;
  const int nkeep = min(keep_first, lo);
  const int nt_keep = (nkeep + KT - 1) / KT;
  const int nt = nt_keep + (i - lo) / KT + 1;
  const int tps = (nt + nsplit - 1) / nsplit;
  const int ti_lo = blockIdx.z * tps, ti_hi = min(nt, ti_lo + tps);
  const bool qok = ql < nh;
  const int head = g * nh + (qok ? ql : 0);
  // the token's queries: read once by the whole block (16-byte loads over the heads' contiguous rows),
  // rounded to bf16 into the key tile's LDS, and from there into every wave's fragments
  bf16x8 Qf[D / 16];
  {
    const float* qb = q + (size_t)t * ldq + (size_t)g * nh * D;
    for (int e = threadIdx.x; e < 32 * (D / 4); e += 256) {
      const int hh = e / (D / 4), c4 = e % (D / 4);
      float4 f = make_float4(0.f, 0.f, 0.f, 0.f);
      if (hh < nh) f = *reinterpret_cast<const float4*>(qb + (size_t)hh * D + c4 * 4);
      bf16_t e4[4] = {f_to_bf16(f.x), f_to_bf16(f.y), f_to_bf16(f.z), f_to_bf16(f.w)};
      *reinterpret_cast<uint2*>(Ks + hh * KLD + c4 * 4) = *reinterpret_cast<const uint2*>(e4);
    }
    __syncthreads();
#pragma unroll
    for (int s = 0; s < D / 16; ++s) Qf[s] = *reinterpret_cast<const bf16x8*>(Ks + ql * KLD + 16 * s + h2 * 8);
  }
  floatx16 O[CPW];
#pragma unroll
  for (int c = 0; c < CPW; ++c)
#pragma unroll
    for (int r = 0; r < 16; ++r) O[c][r] = 0.f;
  float m = -1e30f, l = 0.f;
  constexpr int NK = KT * (D / 8) / 256, NV = KT * (DV / 8) / 256;
  static_assert(NK >= 1 && NV >= 1 && KT * (D / 8) % 256 == 0 && KT * (DV / 8) % 256 == 0 && CPW >= 1, "tile pieces per thread");
  uint4 kreg[NK], vreg[NV];
  auto fetch = [&](int ti) {
    const int j0 = ti < nt_keep ? ti * KT : lo + (ti - nt_keep) * KT;
    const int jend = ti < nt_keep ? nkeep : i + 1;
#pragma unroll
    for (int x = 0; x < NK; ++x) {
      const int e = threadIdx.x + 256 * x;
      const int j = j0 + e / (D / 8), seg = e % (D / 8);
      kreg[x] = make_uint4(0, 0, 0, 0);
      if (j < jend) {
        const size_t row = (size_t)table[j / page_size] * page_size + j % page_size;
        kreg[x] = *reinterpret_cast<const uint4*>(kc + row * ldk + (size_t)g * D + seg * 8);
      }
    }
#pragma unroll
    for (int x = 0; x < NV; ++x) {
      const int e = threadIdx.x + 256 * x;
      const int j = j0 + e % KT, seg = e / KT;
      vreg[x] = make_uint4(0, 0, 0, 0);
      if (j < jend) {
        const size_t row = (size_t)table[j / page_size] * page_size + j % page_size;
        vreg[x] = *reinterpret_cast<const uint4*>(vc + row * ldv + (size_t)g * DV + seg * 8);
      }
    }
  };
  if (ti_lo < ti_hi) fetch(ti_lo);
  for (int ti = ti_lo; ti < ti_hi; ++ti) {
    const bool kept = ti < nt_keep;
    const int j0 = kept ? ti * KT : lo + (ti - nt_keep) * KT;
    const int jend = kept ? nkeep : i + 1;
    __syncthreads();
#pragma unroll
    for (int x = 0; x < NK; ++x) {
      const int e = threadIdx.x + 256 * x;
      *reinterpret_cast<uint4*>(Ks + (e / (D / 8)) * KLD + (e % (D / 8)) * 8) = kreg[x];
    }
#pragma unroll
    for (int x = 0; x < NV; ++x) {
      const int e = threadIdx.x + 256 * x;
      const int kk = e % KT, seg = e / KT;
      const bf16_t* ev = reinterpret_cast<const bf16_t*>(&vreg[x]);
#pragma unroll
      for (int y = 0; y < 8; ++y) Vt[(seg * 8 + y) * PLD + kk] = ev[y];
    }
    __syncthreads();
    if (ti + 1 < ti_hi) fetch(ti + 1);
    floatx16 S;
#pragma unroll
    for (int r = 0; r < 16; ++r) S[r] = 0.f;
#pragma unroll
    for (int s = 0; s < D / 16; ++s) {
      const bf16x8 kf = *reinterpret_cast<const bf16x8*>(Ks + ql * KLD + 16 * s + h2 * 8);
      S = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, Qf[s], S, 0, 0, 0);
    }
    float p[16];
    float mt = -1e30f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int j = j0 + 8 * (r >> 2) + 4 * h2 + (r & 3);
      const bool vis = qok && j < jend;            // (every key of a tile below jend is visible: j <= i, inside the window or kept)
      p[r] = vis ? S[r] * scale : -1e30f;
      mt = fmaxf(mt, p[r]);
    }
    mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
    mt = fmaxf(mt, m);
    float ps = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      p[r] = p[r] > -1e29f ? __expf(p[r] - mt) : 0.f;
      ps += p[r];
    }
    ps += __shfl_xor(ps, 32, 64);
    const float corr = __expf(m - mt);
    l = l * corr + ps;
    m = mt;
#pragma unroll
    for (int c = 0; c < CPW; ++c)
#pragma unroll
      for (int r = 0; r < 16; ++r) O[c][r] *= corr;
    bf16_t* ph = Ps[wave][0] + ql * PLD;
    bf16_t* pl = Ps[wave][1] + ql * PLD;
#pragma unroll
    for (int rg = 0; rg < 4; ++rg) {
      bf16_t hi[4], lw[4];
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        hi[x] = f_to_bf16(p[4 * rg + x]);
        lw[x] = f_to_bf16(p[4 * rg + x] - bf16_to_f(hi[x]));
      }
      *reinterpret_cast<uint2*>(ph + 8 * rg + 4 * h2) = *reinterpret_cast<const uint2*>(hi);
      *reinterpret_cast<uint2*>(pl + 8 * rg + 4 * h2) = *reinterpret_cast<const uint2*>(lw);
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int ks = 0; ks < KT / 16; ++ks) {
      const bf16x8 bh = *reinterpret_cast<const bf16x8*>(ph + 16 * ks + 8 * h2);
      const bf16x8 bl = *reinterpret_cast<const bf16x8*>(pl + 16 * ks + 8 * h2);
#pragma unroll
      for (int c = 0; c < CPW; ++c) {
        const bf16x8 vf = *reinterpret_cast<const bf16x8*>(Vt + (32 * (wave * CPW + c) + ql) * PLD + 16 * ks + 8 * h2);
        O[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, bh, O[c], 0, 0, 0);
        O[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, bl, O[c], 0, 0, 0);
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  if (!qok) return;
  if (nsplit == 1) {
    const float inv = out_scale / l;
    bf16_t* op = out + (size_t)t * ldo + (size_t)head * DV;
#pragma unroll
    for (int c = 0; c < CPW; ++c)
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        bf16_t o4[4];
#pragma unroll
        for (int x = 0; x < 4; ++x) o4[x] = f_to_bf16(O[c][4 * rg + x] * inv);
        *reinterpret_cast<uint2*>(op + 32 * (wave * CPW + c) + 8 * rg + 4 * h2) = *reinterpret_cast<const uint2*>(o4);
      }
  } else {
    float* pp = part + (((size_t)t * H + head) * nsplit + blockIdx.z) * (DV + 4);     // record: values[DV] | maximum | sum | pad
    if (wave == 0 && h2 == 0) { pp[DV] = m; pp[DV + 1] = l; }
#pragma unroll
    for (int c = 0; c < CPW; ++c)
#pragma unroll
      for (int rg = 0; rg < 4; ++rg)
        *reinterpret_cast<float4*>(pp + 32 * (wave * CPW + c) + 8 * rg + 4 * h2) =
            make_float4(O[c][4 * rg], O[c][4 * rg + 1], O[c][4 * rg + 2], O[c][4 * rg + 3]);
  }
}

// -2: shape not served (the caller runs fls_seq_attn_paged)
extern "C" int fls_seq_attn_heads(const void* q, int ldq, const void* kc, int ldk, const void* vc, int ldv, void* out, int ldo,
                                  const int* tok_seq, const int* tok_pos, const int* page_table, int pt_stride, int T, int H,
                                  int G, int d, int dv, float scale, int window, int keep_first, float out_scale, int page_size,
                                  int nsplit, float* part, fls_stream_t s) {
  if (T <= 0) return 0;
  if (G < 1 || H % G || H / G > 32 || page_size < 1 || nsplit < 1 || nsplit > 64 || (nsplit > 1 && part == nullptr) || ldq % 4 || ldo % 4 ||
      ldk % 8 || ldv % 8 || G * d > ldk || G * dv > ldv || (uintptr_t)q % 16 || (uintptr_t)kc % 16 || (uintptr_t)vc % 16 ||
      (uintptr_t)out % 8 || keep_first < 0)
    return -2;
  dim3 grid(T, G, nsplit);
  hipStream_t st = (hipStream_t)s;
#define ATTN_HEADS(DD, DDV)                                                                                                \
  hipLaunchKernelGGL((attn_heads_kernel<DD, DDV>), grid, dim3(256), 0, st, (const float*)q, ldq, (const bf16_t*)kc, ldk,    \
                     (const bf16_t*)vc, ldv, (bf16_t*)out, ldo, tok_seq, tok_pos, page_table, pt_stride, H, G, scale, window, \
                     keep_first, out_scale, page_size, part)
  if (d == 576 && dv == 512) ATTN_HEADS(576, 512);
  else if (d == 320 && dv == 256) ATTN_HEADS(320, 256);
  else if (d == 192 && dv == 128) ATTN_HEADS(192, 128);
  else return -2;
#undef ATTN_HEADS
  SEQ_LAUNCH_CHECK();
  if (nsplit > 1) return seq_attn_merge(part, out, 1, ldo, T, H, dv, nsplit, 0, out_scale, 0, 0.f, nullptr, 0, s);
  return 0;
}
