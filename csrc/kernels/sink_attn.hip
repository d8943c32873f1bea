// Grouped-query softmax attention over a paged cache whose row per token is [K: G x dim | V: G x vdim], for prompt
// portions and single decode tokens alike. A query at position p of its sequence sees the cached positions j <= p
// with p - j < window (window 0: all of them); its score is (q . k_j) * scale + bias[min(p - j, bias_rows - 1), h]
// (bias optional); the softmax denominator holds one more per-head term exp(sink_h) that belongs to no position
// (the running maximum starts at the sink, the running sum at 1). Query and value widths may differ.
//
// Scores, softmax weights and the weighted sum are fp32; storage of q / cache / out is bf16 or fp32.
//
// FMA form (any shape, both storage types): a workgroup of 4 waves owns 4 * RPW rows (a row = one token and one
// of the H / G query heads of ONE key/value head), stages tiles of BK keys and values once in LDS as fp32 (odd row
// stride) and shares them between its rows. Lanes split (key, slice of dim) for the scores, value columns for the
// weighted sum.
#include "common.h"
#include "seq_launchers.h"

namespace die {

namespace {

constexpr int WAVES = 4;

template <bool F32> __device__ __forceinline__ float ldt(const void* p, int64_t i) {
  if constexpr (F32)
    return reinterpret_cast<const float*>(p)[i];
  else
    return bf2f(reinterpret_cast<const bf16_t*>(p)[i]);
}
template <bool F32> __device__ __forceinline__ void stt(void* p, int64_t i, float v) {
  if constexpr (F32)
    reinterpret_cast<float*>(p)[i] = v;
  else
    reinterpret_cast<bf16_t*>(p)[i] = f2bf(v);
}

template <int BK, int CC, int RPW, bool F32>
__global__ void __launch_bounds__(256) sink_attn_kernel(SinkAttnArgs a, int QS, int KS, int VS) {
  constexpr int RW = RPW * WAVES;
  extern __shared__ float smem[];
  float* qs = smem;                 // [RW][QS]
  float* ks = qs + RW * QS;         // [BK][KS]
  float* vs = ks + BK * KS;         // [BK][VS]
  float* ps = vs + BK * VS;         // [RW][BK]
  const int s = blockIdx.y, g = blockIdx.z, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int H = a.heads, G = a.kv_heads, QPG = H / G, D = a.dim, DV = a.vdim;
  const int roww = G * (D + DV);
  const int q0 = a.cu_q ? a.cu_q[s] : s;
  const int nq = a.cu_q ? a.cu_q[s + 1] - q0 : 1;
  const int nrows = nq * QPG, row0 = blockIdx.x * RW;
  if (row0 >= nrows) return;
  const int ctx = a.ctx_lens[s];
  const int last_row = min(row0 + RW, nrows) - 1;
  const int p_first = (int)a.positions[q0 + row0 / QPG], p_last = (int)a.positions[q0 + last_row / QPG];
  const int jlo = a.window > 0 ? max(0, p_first - a.window + 1) : 0;
  const int jhi = min(p_last, ctx - 1);

  for (int r = wave; r < RW; r += WAVES) {
    const int row = row0 + r;
    const bool ok = row < nrows;
    const int64_t t = q0 + (ok ? row / QPG : 0);
    const int h = g * QPG + (ok ? row % QPG : 0);
    for (int d = lane; d < QS; d += 64) qs[r * QS + d] = (ok && d < D) ? ldt<F32>(a.q, (t * H + h) * D + d) : 0.f;
  }

  int prow[RPW], hrow[RPW];
  bool rok[RPW];
  float m[RPW], l[RPW], o[RPW][CC];
#pragma unroll
  for (int i = 0; i < RPW; ++i) {
    const int row = row0 + wave * RPW + i;
    rok[i] = row < nrows;
    prow[i] = rok[i] ? (int)a.positions[q0 + row / QPG] : -1;
    hrow[i] = g * QPG + (rok[i] ? row % QPG : 0);
    const bool has_sink = a.sink != nullptr && rok[i];
    m[i] = has_sink ? a.sink[hrow[i]] : -1e30f;
    l[i] = has_sink ? 1.0f : 0.0f;
#pragma unroll
    for (int c = 0; c < CC; ++c) o[i][c] = 0.f;
  }

  constexpr int NP = 64 / BK;
  const int key = lane % BK, part = lane / BK;
  const int dlen = (D + NP - 1) / NP, d0 = part * dlen, d1 = min(D, d0 + dlen);
  const int* bt = a.block_tables + (int64_t)s * a.bt_stride;

  for (int j0 = jlo; j0 <= jhi; j0 += BK) {
    __syncthreads();
    for (int k = wave; k < BK; k += WAVES) {
      const int j = j0 + k;
      const bool in = j <= jhi;
      const int64_t rowp = in ? ((int64_t)bt[j / a.block_size] * a.block_size + j % a.block_size) * roww : 0;
      for (int d = lane; d < D; d += 64) ks[k * KS + d] = in ? ldt<F32>(a.cache, rowp + g * D + d) : 0.f;
      for (int d = lane; d < DV; d += 64) vs[k * VS + d] = in ? ldt<F32>(a.cache, rowp + G * D + g * DV + d) : 0.f;
    }
    __syncthreads();
    float acc[RPW];
#pragma unroll
    for (int i = 0; i < RPW; ++i) acc[i] = 0.f;
    for (int d = d0; d < d1; ++d) {
      const float kv = ks[key * KS + d];
#pragma unroll
      for (int i = 0; i < RPW; ++i) acc[i] += qs[(wave * RPW + i) * QS + d] * kv;
    }
    const int j = j0 + key;
    float alpha[RPW];
#pragma unroll
    for (int i = 0; i < RPW; ++i) {
      float sc = acc[i];
#pragma unroll
      for (int off = BK; off < 64; off <<= 1) sc += __shfl_xor(sc, off, 64);
      const int n = prow[i] - j;
      const bool valid = rok[i] && j <= jhi && n >= 0 && (a.window <= 0 || n < a.window);
      sc *= a.scale;
      if (valid && a.bias != nullptr) sc += a.bias[(int64_t)min(n, a.bias_rows - 1) * H + hrow[i]];
      sc = valid ? sc : -INFINITY;
      const float mn = fmaxf(m[i], wave_max(sc));
      const float pe = valid ? expf(sc - mn) : 0.f;
      const float psum = wave_sum(part == 0 ? pe : 0.f);
      alpha[i] = expf(m[i] - mn);
      l[i] = l[i] * alpha[i] + psum;
      m[i] = mn;
      if (part == 0) ps[(wave * RPW + i) * BK + key] = pe;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < RPW; ++i) {
#pragma unroll
      for (int c = 0; c < CC; ++c) o[i][c] *= alpha[i];
    }
    for (int k = 0; k < BK; ++k) {
      float vc[CC];
#pragma unroll
      for (int c = 0; c < CC; ++c) vc[c] = (lane + 64 * c < DV) ? vs[k * VS + lane + 64 * c] : 0.f;
#pragma unroll
      for (int i = 0; i < RPW; ++i) {
        const float pk = ps[(wave * RPW + i) * BK + k];
#pragma unroll
        for (int c = 0; c < CC; ++c) o[i][c] += pk * vc[c];
      }
    }
  }

#pragma unroll
  for (int i = 0; i < RPW; ++i) {
    if (!rok[i]) continue;
    const int row = row0 + wave * RPW + i;
    const int64_t t = q0 + row / QPG;
    const float inv = l[i] > 0.f ? 1.0f / l[i] : 0.f;
#pragma unroll
    for (int c = 0; c < CC; ++c) {
      const int col = lane + 64 * c;
      if (col < DV) stt<F32>(a.out, (t * H + hrow[i]) * DV + col, o[i][c] * inv);
    }
  }
}

inline int odd(int x) { return x | 1; }

template <int BK, int CC, int RPW, bool F32> hipError_t launch_one(const SinkAttnArgs& a, hipStream_t s) {
  constexpr int RW = RPW * WAVES;
  const int QS = odd(a.dim), KS = odd(a.dim), VS = odd(a.vdim);
  const size_t lds = sizeof(float) * ((size_t)RW * QS + (size_t)BK * KS + (size_t)BK * VS + (size_t)RW * BK);
  if (lds > 150 * 1024) return hipErrorInvalidValue;
  auto kern = sink_attn_kernel<BK, CC, RPW, F32>;
  if (lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)lds);
    if (e != hipSuccess) return e;
  }
  const int qpg = a.heads / a.kv_heads;
  const int tiles = (a.max_q * qpg + RW - 1) / RW;
  hipLaunchKernelGGL(kern, dim3(tiles, a.num_seqs, a.kv_heads), dim3(256), lds, s, a, QS, KS, VS);
  return hipGetLastError();
}

template <int BK, int RPW, bool F32> hipError_t launch_cc(const SinkAttnArgs& a, hipStream_t s) {
  if (a.vdim <= 64) return launch_one<BK, 1, RPW, F32>(a, s);
  if (a.vdim <= 128) return launch_one<BK, 2, RPW, F32>(a, s);
  if (a.vdim <= 256) return launch_one<BK, 4, RPW, F32>(a, s);
  return hipErrorInvalidValue;
}

template <bool F32> hipError_t launch_fma(const SinkAttnArgs& a, hipStream_t s) {
  const int qpg = a.heads / a.kv_heads;
  // few rows per (sequence, key/value head): one row per wave, smaller key tiles
  if (a.max_q * qpg <= 4) return launch_cc<32, 1, F32>(a, s);
  if (a.dim + a.vdim > 384) return launch_cc<32, 4, F32>(a, s);
  return launch_cc<64, 4, F32>(a, s);
}

}  // namespace

bool sink_attn_uses_mfma(const SinkAttnArgs&) { return false; }

hipError_t launch_sink_attn(const SinkAttnArgs& a, hipStream_t s) {
  if (a.num_seqs == 0 || a.total_q == 0) return hipSuccess;
  if (a.heads < 1 || a.kv_heads < 1 || a.heads % a.kv_heads != 0 || a.dim < 1 || a.dim > 512 || a.vdim < 1 ||
      a.vdim > 256 || a.block_size < 1 || a.max_q < 1 || (a.bias != nullptr && a.bias_rows < 1))
    return hipErrorInvalidValue;
  if (a.impl == 2) return hipErrorInvalidValue;
  return a.f32 ? launch_fma<true>(a, s) : launch_fma<false>(a, s);
}

}  // namespace die
