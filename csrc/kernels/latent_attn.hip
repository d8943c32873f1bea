// Latent (compressed-KV) attention over the paged latent cache, in its absorbed form: every head's query
// is first projected into the latent space (q_lat = W_uk^T q_nope, a batched GEMM outside this file), so
// all heads of a token score against the SAME cached row [latent | rotated shared key part] and the output
// is the weighted sum of the latent rows (W_uv is applied afterwards). One kernel serves prompt chunks and
// single decode tokens: a row is a (token, head) pair, its keys are the cache positions j <= p inside the
// sliding window, and the softmax denominator may hold a per-head sink term exp(sink_h) that has no key
// and no value (running max starts at the sink, running sum at 1).
//
// Scores, softmax weights and the weighted sum are fp32 (FMA); storage of q / cache / out is bf16 or fp32.
// Workgroup = 4 waves x 4 rows. A tile of BK keys is staged once in LDS as fp32 (row stride odd: a lane per
// key reads conflict-free; a lane per column too) and shared by the 16 rows. Lanes split (key, part of the
// score dimension); the rotary part of q is rotated while it is loaded.
#include "common.h"
#include "mix_launchers.h"

namespace die {

namespace {

constexpr int RPW = 4, WAVES = 4, RW = RPW * WAVES;

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

template <int BK, int CC, bool F32>
__global__ void __launch_bounds__(256) latent_attn_kernel(LatentAttnArgs a, int QS, int KS) {
  extern __shared__ float smem[];
  float* qs = smem;                 // [RW][QS]
  float* ks = qs + RW * QS;         // [BK][KS]
  float* ps = ks + BK * KS;         // [WAVES][RPW][BK]
  const int s = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int H = a.heads, R = a.sh.rank, Dk = a.sh.rank + a.sh.rot_dim;
  const int q0 = a.cu_q ? a.cu_q[s] : s;
  const int nq = a.cu_q ? a.cu_q[s + 1] - q0 : 1;
  const int nrows = nq * H, row0 = blockIdx.x * RW;
  if (row0 >= nrows) return;
  const int ctx = a.ctx_lens[s];
  const int last_row = min(row0 + RW, nrows) - 1;
  const int p_first = (int)a.positions[q0 + row0 / H], p_last = (int)a.positions[q0 + last_row / H];
  const int jlo = a.window > 0 ? max(0, p_first - a.window + 1) : 0;
  const int jhi = min(p_last, ctx - 1);

  // queries -> LDS (fp32), the rotary part rotated by the row's position
  for (int r = wave; r < RW; r += WAVES) {
    const int row = row0 + r;
    const bool ok = row < nrows;
    const int tl = ok ? row / H : 0, h = ok ? row % H : 0;
    const int64_t t = q0 + tl;
    const float p = ok ? (float)a.positions[t] : 0.f;
    const int64_t ql = ((int64_t)h * a.total_q + t) * R;
    const int64_t qr = t * a.q_stride + (int64_t)h * a.q_hstride;
    for (int d = lane; d < QS; d += 64) {
      float v = 0.f;
      if (ok && d < R) {
        v = ldt<F32>(a.q_lat, ql + d);
      } else if (ok && d < Dk) {
        const int dd = d - R, i = dd >> 1;
        if (i < a.sh.rot_pairs) {
          const float u = ldt<F32>(a.q_rot, qr + 2 * i), w = ldt<F32>(a.q_rot, qr + 2 * i + 1);
          float sn, cs;
          sincosf(p * a.sh.inv_freq[i], &sn, &cs);
          v = (dd & 1) ? w * cs + u * sn : u * cs - w * sn;
        } else {
          v = ldt<F32>(a.q_rot, qr + dd);
        }
      }
      qs[r * QS + d] = v;
    }
  }

  int prow[RPW];
  bool rok[RPW];
  float m[RPW], l[RPW], o[RPW][CC];
#pragma unroll
  for (int i = 0; i < RPW; ++i) {
    const int row = row0 + wave * RPW + i;
    rok[i] = row < nrows;
    prow[i] = rok[i] ? (int)a.positions[q0 + row / H] : -1;
    const bool has_sink = a.sink != nullptr && rok[i];
    m[i] = has_sink ? a.sink[row % H] : -1e30f;
    l[i] = has_sink ? 1.0f : 0.0f;
#pragma unroll
    for (int c = 0; c < CC; ++c) o[i][c] = 0.f;
  }

  constexpr int NP = 64 / BK;
  const int key = lane % BK, part = lane / BK;
  const int dlen = (Dk + NP - 1) / NP, d0 = part * dlen, d1 = min(Dk, d0 + dlen);
  const int* bt = a.block_tables + (int64_t)s * a.bt_stride;

  for (int j0 = jlo; j0 <= jhi; j0 += BK) {
    __syncthreads();  // the previous tile (and, first, the queries) are no longer / now in LDS
    for (int k = wave; k < BK; k += WAVES) {
      const int j = j0 + k;
      const bool in = j <= jhi;
      const int64_t rowp = in ? ((int64_t)bt[j / a.block_size] * a.block_size + j % a.block_size) * Dk : 0;
      for (int d = lane; d < Dk; d += 64) ks[k * KS + d] = in ? ldt<F32>(a.cache, rowp + d) : 0.f;
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
      const bool valid = rok[i] && j <= jhi && j <= prow[i] && (a.window <= 0 || prow[i] - j < a.window);
      sc = valid ? sc * a.scale : -INFINITY;
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
      float kvc[CC];
#pragma unroll
      for (int c = 0; c < CC; ++c) kvc[c] = (lane + 64 * c < R) ? ks[k * KS + lane + 64 * c] : 0.f;
#pragma unroll
      for (int i = 0; i < RPW; ++i) {
        const float pk = ps[(wave * RPW + i) * BK + k];
#pragma unroll
        for (int c = 0; c < CC; ++c) o[i][c] += pk * kvc[c];
      }
    }
  }

#pragma unroll
  for (int i = 0; i < RPW; ++i) {
    if (!rok[i]) continue;
    const int row = row0 + wave * RPW + i;
    const int64_t t = q0 + row / H;
    const int h = row % H;
    const float inv = l[i] > 0.f ? 1.0f / l[i] : 0.f;
#pragma unroll
    for (int c = 0; c < CC; ++c) {
      const int col = lane + 64 * c;
      if (col < R) stt<F32>(a.out, ((int64_t)h * a.total_q + t) * R + col, o[i][c] * inv);
    }
  }
}

constexpr int LDS_MAX = 128 * 1024;

inline size_t lds_bytes(int bk, int qs, int ksd) { return sizeof(float) * ((size_t)RW * qs + (size_t)bk * ksd + (size_t)RW * bk); }

template <int BK, int CC, bool F32>
hipError_t launch_one(const LatentAttnArgs& a, int qs, int ksd, dim3 grid, hipStream_t s) {
  static bool attr_set = false;  // once per instantiation; hipFuncSetAttribute is not a stream operation
  auto* fn = latent_attn_kernel<BK, CC, F32>;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       LDS_MAX);
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  hipLaunchKernelGGL(fn, grid, dim3(256), lds_bytes(BK, qs, ksd), s, a, qs, ksd);
  return hipGetLastError();
}

template <int BK, bool F32>
hipError_t launch_cc(const LatentAttnArgs& a, int qs, int ksd, dim3 grid, hipStream_t s) {
  const int r = a.sh.rank;
  if (r <= 128) return launch_one<BK, 2, F32>(a, qs, ksd, grid, s);
  if (r <= 512) return launch_one<BK, 8, F32>(a, qs, ksd, grid, s);
  if (r <= 1024) return launch_one<BK, 16, F32>(a, qs, ksd, grid, s);
  return hipErrorInvalidValue;
}

template <bool F32> hipError_t launch_bk(const LatentAttnArgs& a, hipStream_t s) {
  const int dk = a.sh.rank + a.sh.rot_dim;
  const int qs = (dk + 3) & ~3, ksd = dk | 1;
  const dim3 grid((unsigned)(((int64_t)a.max_q * a.heads + RW - 1) / RW), (unsigned)a.num_seqs);
  if (lds_bytes(64, qs, ksd) <= 64 * 1024) return launch_cc<64, F32>(a, qs, ksd, grid, s);
  if (lds_bytes(32, qs, ksd) <= LDS_MAX) return launch_cc<32, F32>(a, qs, ksd, grid, s);
  if (lds_bytes(16, qs, ksd) <= LDS_MAX) return launch_cc<16, F32>(a, qs, ksd, grid, s);
  return hipErrorInvalidValue;
}

}  // namespace

hipError_t launch_latent_attn(const LatentAttnArgs& a, hipStream_t s) {
  if (a.num_seqs == 0 || a.total_q == 0) return hipSuccess;
  if (a.heads < 1 || a.sh.rank < 1 || a.sh.rot_dim < 0 || a.sh.rot_pairs * 2 > a.sh.rot_dim || a.block_size < 1 ||
      a.max_q < 1)
    return hipErrorInvalidValue;
  return a.f32 ? launch_bk<true>(a, s) : launch_bk<false>(a, s);
}

}  // namespace die
