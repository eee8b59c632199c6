// Latent attention over a paged cache that holds, per token, one normed latent vector (rank) and one
// rotated key part (rot) shared by all heads. The per-head key and value up-projections are absorbed
// into the query and the output (q' = W_uk^T q, out = W_uv (sum_j p_j c_j)), so prompt portions and
// single decoded tokens run the same kernel on the cached rows alone:
//   score(t, h, j) = scale * (q'[t][h] . c_j + rope(q_rot[t][h]) . k_rot_j),   j <= position(t)
//   ol[t][h]       = sum_j softmax_j(score) c_j
// latent_write: RMS norm of the latent (fp32 statistics) + interleaved-pair rotation of the shared key
// part + the paged store, one launch. Angles are position * inv_freq in fp32 with full-range sin / cos.
// latent_attn: one workgroup per (token, group of heads); key tiles of 16 rows staged in LDS as fp32,
// scores, running max / sum and the weighted latent sum all in fp32.
#include "common.h"
#include "seq_launchers.h"

namespace vgate {
namespace {

__device__ __forceinline__ float ldx(const void* p, int64_t i, int f32) {
  return f32 ? reinterpret_cast<const float*>(p)[i] : bf2f(reinterpret_cast<const bf16_t*>(p)[i]);
}
__device__ __forceinline__ void stx(void* p, int64_t i, int f32, float v) {
  if (f32) reinterpret_cast<float*>(p)[i] = v;
  else reinterpret_cast<bf16_t*>(p)[i] = f2bf(v);
}

__global__ __launch_bounds__(256) void latent_write_kernel(LatentArgs a, const void* __restrict__ kv, int64_t ldkv,
                                                            const float* __restrict__ w, float eps) {
  __shared__ float red[16];
  const int t = blockIdx.x;
  const int slot = a.slots[t];
  if (slot < 0) return;  // uniform per block
  const int64_t src = (int64_t)t * ldkv;
  const int64_t dst = (int64_t)slot * (a.rank + a.rot);
  float ss = 0.f;
  for (int c = threadIdx.x; c < a.rank; c += blockDim.x) {
    const float v = ldx(kv, src + c, a.f32);
    ss = fmaf(v, v, ss);
  }
  ss = block_reduce_sum(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)a.rank + eps);
  for (int c = threadIdx.x; c < a.rank; c += blockDim.x)
    stx(a.cache, dst + c, a.f32, ldx(kv, src + c, a.f32) * inv * w[c]);
  const float pos = (float)a.positions[t];
  for (int i = threadIdx.x; i < a.rot; i += blockDim.x) {
    float o;
    if (i < a.rot_dims) {
      const float ang = pos * a.inv_freq[i >> 1];
      const float cs = cosf(ang), sn = sinf(ang);
      const float u = ldx(kv, src + a.rank + (i & ~1), a.f32), v = ldx(kv, src + a.rank + (i | 1), a.f32);
      o = (i & 1) ? (v * cs + u * sn) : (u * cs - v * sn);
    } else {
      o = ldx(kv, src + a.rank + i, a.f32);
    }
    stx(a.cache, dst + a.rank + i, a.f32, o);
  }
}

__global__ __launch_bounds__(256) void latent_qrope_kernel(LatentArgs a, const void* __restrict__ q, int H, int dim,
                                                            void* __restrict__ qa) {
  const int t = blockIdx.x;
  const float pos = (float)a.positions[t];
  for (int e = threadIdx.x; e < H * a.rot; e += blockDim.x) {
    const int h = e / a.rot, i = e % a.rot;
    const int64_t src = ((int64_t)t * H + h) * (dim + a.rot) + dim;
    float o;
    if (i < a.rot_dims) {
      const float ang = pos * a.inv_freq[i >> 1];
      const float cs = cosf(ang), sn = sinf(ang);
      const float u = ldx(q, src + (i & ~1), a.f32), v = ldx(q, src + (i | 1), a.f32);
      o = (i & 1) ? (v * cs + u * sn) : (u * cs - v * sn);
    } else {
      o = ldx(q, src + i, a.f32);
    }
    stx(qa, ((int64_t)t * H + h) * (a.rank + a.rot) + a.rank + i, a.f32, o);
  }
}

constexpr int KT = 16;      // keys per tile
constexpr int MAXACC = 16;  // latent outputs per thread: heads-per-block * rank <= 256 * MAXACC

__global__ __launch_bounds__(256) void latent_attn_kernel(LatentArgs a, const void* __restrict__ qa, int H, int HC,
                                                           float scale, const int32_t* __restrict__ block_tables,
                                                           int max_blocks, int page,
                                                           const int32_t* __restrict__ context_lens,
                                                           const int32_t* __restrict__ query_start, int S,
                                                           void* __restrict__ ol) {
  extern __shared__ float lds[];
  const int E = a.rank + a.rot, EP = E + 1;
  float* qs = lds;                  // [HC][EP]
  float* ks = qs + HC * EP;         // [KT][EP]
  float* sc = ks + KT * EP;         // [HC][KT] scores, then weights
  float* mrun = sc + HC * KT;       // [HC]
  float* lrun = mrun + HC;          // [HC]
  float* alpha = lrun + HC;         // [HC]
  const int t = blockIdx.x;
  if (t >= query_start[S]) return;
  int lo = 0, hi = S - 1;           // the sequence of token t: query_start[s] <= t < query_start[s + 1]
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (query_start[mid] <= t) lo = mid; else hi = mid - 1;
  }
  const int s = lo;
  const int nkeys = context_lens[s] - (query_start[s + 1] - t) + 1;
  const int h0 = blockIdx.y * HC;
  const int nh = min(HC, H - h0);
  const int tid = threadIdx.x;
  for (int e = tid; e < nh * E; e += 256) {
    const int h = e / E, c = e % E;
    qs[h * EP + c] = ldx(qa, ((int64_t)t * H + h0 + h) * E + c, a.f32);
  }
  if (tid < HC) { mrun[tid] = -INFINITY; lrun[tid] = 0.f; alpha[tid] = 1.f; }
  float acc[MAXACC];
#pragma unroll
  for (int i = 0; i < MAXACC; ++i) acc[i] = 0.f;
  const int32_t* bt = block_tables + (int64_t)s * max_blocks;
  for (int j0 = 0; j0 < nkeys; j0 += KT) {
    __syncthreads();  // previous tile fully consumed (and q / running stats written)
    for (int e = tid; e < KT * E; e += 256) {
      const int jj = e / E, c = e % E;
      const int kj = j0 + jj;
      float v = 0.f;
      if (kj < nkeys) {
        const int64_t row = (int64_t)bt[kj / page] * page + kj % page;
        v = ldx(a.cache, row * E + c, a.f32);
      }
      ks[jj * EP + c] = v;
    }
    __syncthreads();
    {  // scores: two threads per (head, key), each half of the dot product
      const int wi = tid >> 1, half = tid & 1;
      float d = 0.f;
      const bool on = wi < nh * KT;
      const int h = on ? wi / KT : 0, jj = on ? wi % KT : 0;
      if (on) {
        const int c0 = half ? (E >> 1) : 0, c1 = half ? E : (E >> 1);
        const float* qp = qs + h * EP;
        const float* kp = ks + jj * EP;
        for (int c = c0; c < c1; ++c) d = fmaf(qp[c], kp[c], d);
      }
      d += __shfl_xor(d, 1, 64);
      if (on && half == 0) sc[h * KT + jj] = (j0 + jj < nkeys) ? d * scale : -INFINITY;
    }
    __syncthreads();
    if (tid < nh) {
      const float m0 = mrun[tid];
      float m1 = m0;
      for (int jj = 0; jj < KT; ++jj) m1 = fmaxf(m1, sc[tid * KT + jj]);
      const float al = expf(m0 - m1);  // m0 = -inf on the first tile: 0
      float l = lrun[tid] * al;
      for (int jj = 0; jj < KT; ++jj) {
        const float pj = expf(sc[tid * KT + jj] - m1);
        sc[tid * KT + jj] = pj;
        l += pj;
      }
      mrun[tid] = m1; lrun[tid] = l; alpha[tid] = al;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < MAXACC; ++i) {
      const int o = tid + i * 256;
      if (o < nh * a.rank) {
        const int h = o / a.rank, c = o % a.rank;
        float v = acc[i] * alpha[h];
        const float* pp = sc + h * KT;
#pragma unroll
        for (int jj = 0; jj < KT; ++jj) v = fmaf(pp[jj], ks[jj * EP + c], v);
        acc[i] = v;
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < MAXACC; ++i) {
    const int o = tid + i * 256;
    if (o < nh * a.rank) {
      const int h = o / a.rank, c = o % a.rank;
      stx(ol, ((int64_t)t * H + h0 + h) * a.rank + c, a.f32, acc[i] / lrun[h]);
    }
  }
}

}  // namespace

void launch_latent_write(const LatentArgs& a, const void* kv, int64_t ldkv, const float* w, float eps, hipStream_t st) {
  if (a.T <= 0) return;
  hipLaunchKernelGGL(latent_write_kernel, dim3(a.T), dim3(256), 0, st, a, kv, ldkv, w, eps);
}

void launch_latent_qrope(const LatentArgs& a, const void* q, int H, int dim, void* qa, hipStream_t st) {
  if (a.T <= 0) return;
  hipLaunchKernelGGL(latent_qrope_kernel, dim3(a.T), dim3(256), 0, st, a, q, H, dim, qa);
}

void launch_latent_attn(const LatentArgs& a, const void* qa, int H, float scale, const int32_t* block_tables,
                        int max_blocks, int page, const int32_t* context_lens, const int32_t* query_start, int S,
                        void* ol, hipStream_t st) {
  if (a.T <= 0 || S <= 0) return;
  const int E = a.rank + a.rot;
  int HC = H < 8 ? H : 8;
  while (HC > 1 && (HC * a.rank > 256 * MAXACC || (size_t)(HC + KT) * (E + 1) * 4 > 56 * 1024)) --HC;
  const size_t lds = ((size_t)(HC + KT) * (E + 1) + HC * KT + 3 * HC) * sizeof(float);
  hipLaunchKernelGGL(latent_attn_kernel, dim3(a.T, (H + HC - 1) / HC), dim3(256), lds, st, a, qa, H, HC, scale,
                     block_tables, max_blocks, page, context_lens, query_start, S, ol);
}

}  // namespace vgate
