// Grouped-query attention over a sliding window of a paged key/value cache, optionally with pooled
// blocks: every block of P tokens that lies wholly before the window is seen through one row, the mean
// of its cached keys and the mean of its cached values. Caches (activation dtype):
//   kc [pages][G][page][D], vc [pages][G][page][V]       token rows
//   kp [pages][G][NP][D],   vp [pages][G][NP][V]         pooled rows, NP = ceil(page / P): block b's row
//                                                        lives in the page of its last position e = b P + P - 1,
//                                                        at index (e mod page) / P
// window_write  one workgroup per token: query / key RMS norm (per head or over the whole projection,
//               fp32 statistics), interleaved-pair rotation of the leading rot_dims entries of every head
//               (angle = position * inv_freq in fp32, full-range sin / cos), values optionally turned over
//               all of V, the paged stores, and the prepared query rows.
// window_pool   one workgroup per token whose position completes a block: fp32 mean of the block's P
//               cached rows, in position order, into the pooled row. It runs after window_write of the
//               same step, so a block completed inside a prompt portion reads rows of that portion too.
// window_attn   one workgroup per (token, key/value head, chunk of its query heads): the keys a query
//               sees are numbered pooled rows first, then window tokens; tiles of 16 of them are staged in
//               LDS as fp32; scores, running max / sum and the weighted value sum are fp32 FMA. A sink
//               starts the running max at its logit and the running sum at 1. With turned values the
//               normalised output is turned back by the query's position before it is stored.
// Every row of every kernel depends only on its own sequence's cache rows, in an order fixed by the
// position, so results do not depend on how a prompt is cut or what else is in the batch.
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

__device__ __forceinline__ int seq_of_token(const int32_t* query_start, int S, int t) {
  int lo = 0, hi = S - 1;  // query_start[s] <= t < query_start[s + 1]
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (query_start[mid] <= t) lo = mid; else hi = mid - 1;
  }
  return lo;
}

__global__ __launch_bounds__(256) void window_write_kernel(WindowArgs a, const void* __restrict__ q, int64_t ldq,
                                                            const void* __restrict__ k, int64_t ldk,
                                                            const void* __restrict__ v, int64_t ldv,
                                                            const float* __restrict__ qw, const float* __restrict__ kw,
                                                            float eps, int norm_all, void* __restrict__ q_out) {
  extern __shared__ float lds[];
  const int H = a.H, G = a.G, D = a.D, V = a.V;
  float* xs = lds;                    // [(H + G) * D] q heads then k heads
  float* inv = xs + (H + G) * D;      // [H + G]
  const int t = blockIdx.x;
  const int slot = a.slots[t];
  if (slot < 0) return;  // padding row (uniform per block)
  const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63;
  for (int e = tid; e < H * D; e += 256) xs[e] = ldx(q, (int64_t)t * ldq + e, a.f32);
  for (int e = tid; e < G * D; e += 256) xs[H * D + e] = ldx(k, (int64_t)t * ldk + e, a.f32);
  __syncthreads();
  for (int h = wv; h < H + G; h += 4) {  // sum of squares per head
    float ss = 0.f;
    for (int d = lane; d < D; d += 64) ss = fmaf(xs[h * D + d], xs[h * D + d], ss);
    ss = wave_reduce_sum(ss);
    if (lane == 0) inv[h] = ss;
  }
  __syncthreads();
  if (qw != nullptr) {
    float mine = 0.f;
    if (norm_all) {
      float sq = 0.f, sk = 0.f;
      for (int h = 0; h < H; ++h) sq += inv[h];
      for (int h = 0; h < G; ++h) sk += inv[H + h];
      if (tid < H + G) mine = 1.f / sqrtf((tid < H ? sq / (float)(H * D) : sk / (float)(G * D)) + eps);
    } else if (tid < H + G) {
      mine = 1.f / sqrtf(inv[tid] / (float)D + eps);
    }
    __syncthreads();
    if (tid < H + G) inv[tid] = mine;
    __syncthreads();
  }
  const float pos = (float)a.positions[t];
  const int page = a.page;
  const int64_t pg = slot / page, off = slot % page;
  for (int e = tid; e < (H + G) * D; e += 256) {
    const int h = e / D, i = e % D;
    const bool isq = h < H;
    const float* w = isq ? qw : kw;
    const int wo = norm_all ? (isq ? h : h - H) * D : 0;
    const float sc = w != nullptr ? inv[h] : 1.f;
    float o;
    if (i < a.rot_dims) {
      const int i0 = i & ~1, i1 = i | 1;
      const float x0 = xs[h * D + i0] * sc * (w ? w[wo + i0] : 1.f), x1 = xs[h * D + i1] * sc * (w ? w[wo + i1] : 1.f);
      const float ang = pos * a.inv_freq[i >> 1];
      const float cs = cosf(ang), sn = sinf(ang);
      o = (i & 1) ? (x1 * cs + x0 * sn) : (x0 * cs - x1 * sn);
    } else {
      o = xs[h * D + i] * sc * (w ? w[wo + i] : 1.f);
    }
    if (isq) stx(q_out, (int64_t)t * H * D + e, a.f32, o);
    else stx(a.kc, ((pg * G + (h - H)) * page + off) * D + i, a.f32, o);
  }
  const int vrot = a.v_freq != nullptr ? 2 * (V / 2) : 0;
  for (int e = tid; e < G * V; e += 256) {
    const int g = e / V, i = e % V;
    float o;
    if (i < vrot) {
      const float x0 = ldx(v, (int64_t)t * ldv + g * V + (i & ~1), a.f32), x1 = ldx(v, (int64_t)t * ldv + g * V + (i | 1), a.f32);
      const float ang = pos * a.v_freq[i >> 1];
      const float cs = cosf(ang), sn = sinf(ang);
      o = (i & 1) ? (x1 * cs + x0 * sn) : (x0 * cs - x1 * sn);
    } else {
      o = ldx(v, (int64_t)t * ldv + e, a.f32);
    }
    stx(a.vc, ((pg * G + g) * page + off) * V + i, a.f32, o);
  }
}

__global__ __launch_bounds__(256) void window_pool_kernel(WindowArgs a) {
  const int t = blockIdx.x;
  if (t >= a.query_start[a.S]) return;
  const int e = a.positions[t], P = a.pool;
  if ((e + 1) % P != 0) return;  // uniform per block
  const int s = seq_of_token(a.query_start, a.S, t);
  const int32_t* bt = a.block_tables + (int64_t)s * a.max_blocks;
  const int G = a.G, D = a.D, V = a.V, page = a.page;
  const int64_t dpg = bt[e / page];
  const int drow = (e % page) / P;
  for (int x = threadIdx.x; x < G * (D + V); x += blockDim.x) {
    const bool isk = x < G * D;
    const int y = isk ? x : x - G * D;
    const int w = isk ? D : V;
    const int g = y / w, i = y % w;
    const void* src = isk ? a.kc : a.vc;
    float sum = 0.f;
    for (int j = e + 1 - P; j <= e; ++j)
      sum += ldx(src, (((int64_t)bt[j / page] * G + g) * page + j % page) * w + i, a.f32);
    stx(isk ? a.kp : a.vp, ((dpg * G + g) * a.npool + drow) * w + i, a.f32, sum / (float)P);
  }
}

constexpr int KT = 16;      // keys per tile
constexpr int MAXACC = 8;   // outputs per thread: heads-per-block * V <= 256 * MAXACC

__global__ __launch_bounds__(256) void window_attn_kernel(WindowArgs a, const void* __restrict__ q, int HC, float scale,
                                                           void* __restrict__ out) {
  extern __shared__ float lds[];
  const int D = a.D, V = a.V, DP = D + 1, VP = V + 1, G = a.G, page = a.page;
  float* qs = lds;                  // [HC][DP]
  float* ks = qs + HC * DP;         // [KT][DP]
  float* vs = ks + KT * DP;         // [KT][VP]
  float* sc = vs + KT * VP;         // [HC][KT] scores, then weights
  float* mrun = sc + HC * KT;       // [HC]
  float* lrun = mrun + HC;          // [HC]
  float* alpha = lrun + HC;         // [HC]
  float* os = alpha + HC;           // [HC][V] normalised outputs (for the turn back)
  const int t = blockIdx.x;
  if (t >= a.query_start[a.S]) return;
  const int s = seq_of_token(a.query_start, a.S, t);
  const int pos = a.context_lens[s] - (a.query_start[s + 1] - t);  // position of token t
  const int g = blockIdx.y;
  const int rep = a.H / G;
  const int r0 = blockIdx.z * HC;          // first query head of the group handled here
  const int nh = min(HC, rep - r0);
  const int h0 = g * rep + r0;
  const int tid = threadIdx.x;
  const int lo = max(0, pos - a.window + 1);
  const int nb = a.pool > 0 ? max(0, pos - a.window + 1) / a.pool : 0;  // pooled blocks wholly before the window
  const int nkeys = nb + (pos - lo + 1);
  for (int e = tid; e < nh * D; e += 256) qs[(e / D) * DP + e % D] = ldx(q, ((int64_t)t * a.H + h0) * D + e, a.f32);
  if (tid < HC) {
    const bool sk = a.sink != nullptr && tid < nh;
    mrun[tid] = sk ? a.sink[h0 + tid] : -INFINITY;
    lrun[tid] = sk ? 1.f : 0.f;
    alpha[tid] = 1.f;
  }
  float acc[MAXACC];
#pragma unroll
  for (int i = 0; i < MAXACC; ++i) acc[i] = 0.f;
  const int32_t* bt = a.block_tables + (int64_t)s * a.max_blocks;
  for (int j0 = 0; j0 < nkeys; j0 += KT) {
    __syncthreads();  // previous tile fully consumed (and q / running stats written)
    for (int e = tid; e < KT * (D + V); e += 256) {
      const int jj = e / (D + V), c = e % (D + V);
      const int kj = j0 + jj;
      float val = 0.f;
      if (kj < nkeys) {
        const bool isk = c < D;
        const int ci = isk ? c : c - D, w = isk ? D : V;
        if (kj < nb) {   // pooled row of block kj
          const int e1 = kj * a.pool + a.pool - 1;
          const int64_t row = ((int64_t)bt[e1 / page] * G + g) * a.npool + (e1 % page) / a.pool;
          val = ldx(isk ? a.kp : a.vp, row * w + ci, a.f32);
        } else {
          const int j = lo + kj - nb;
          const int64_t row = ((int64_t)bt[j / page] * G + g) * page + j % page;
          val = ldx(isk ? a.kc : a.vc, row * w + ci, a.f32);
        }
      }
      if (c < D) ks[jj * DP + c] = val; else vs[jj * VP + c - D] = val;
    }
    __syncthreads();
    {  // scores: two threads per (head, key), each half of the dot product
      const int wi = tid >> 1, half = tid & 1;
      float d = 0.f;
      const bool on = wi < nh * KT;
      const int h = on ? wi / KT : 0, jj = on ? wi % KT : 0;
      if (on) {
        const int c0 = half ? (D >> 1) : 0, c1 = half ? D : (D >> 1);
        const float* qp = qs + h * DP;
        const float* kp = ks + jj * DP;
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
      if (o < nh * V) {
        const int h = o / V, c = o % V;
        float x = acc[i] * alpha[h];
        const float* pp = sc + h * KT;
#pragma unroll
        for (int jj = 0; jj < KT; ++jj) x = fmaf(pp[jj], vs[jj * VP + c], x);
        acc[i] = x;
      }
    }
  }
  __syncthreads();
  if (a.v_freq == nullptr) {
#pragma unroll
    for (int i = 0; i < MAXACC; ++i) {
      const int o = tid + i * 256;
      if (o < nh * V) stx(out, ((int64_t)t * a.H + h0) * V + o, a.f32, acc[i] / lrun[o / V]);
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < MAXACC; ++i) {
    const int o = tid + i * 256;
    if (o < nh * V) os[o] = acc[i] / lrun[o / V];
  }
  __syncthreads();
  const int vrot = 2 * (V / 2);
  const float fp = -(float)pos;
  for (int o = tid; o < nh * V; o += 256) {
    const int h = o / V, i = o % V;
    float y = os[o];
    if (i < vrot) {
      const float x0 = os[h * V + (i & ~1)], x1 = os[h * V + (i | 1)];
      const float ang = fp * a.v_freq[i >> 1];
      const float cs = cosf(ang), sn = sinf(ang);
      y = (i & 1) ? (x1 * cs + x0 * sn) : (x0 * cs - x1 * sn);
    }
    stx(out, ((int64_t)t * a.H + h0) * V + o, a.f32, y);
  }
}

int heads_per_block(const WindowArgs& a) {
  const int rep = a.H / a.G;
  int HC = rep < 8 ? rep : 8;
  auto lds = [&](int hc) { return window_attn_lds_bytes(a, hc); };
  while (HC > 1 && (HC * a.V > 256 * MAXACC || lds(HC) > 60 * 1024)) --HC;
  return HC;
}

}  // namespace

size_t window_attn_lds_bytes(const WindowArgs& a, int HC) {
  return ((size_t)HC * (a.D + 1) + (size_t)KT * (a.D + 1) + (size_t)KT * (a.V + 1) + HC * KT + 3 * HC + (size_t)HC * a.V) *
         sizeof(float);
}

bool window_attn_fits(const WindowArgs& a) {
  return a.V <= 256 * MAXACC && window_attn_lds_bytes(a, 1) <= 60 * 1024 &&
         (size_t)((a.H + a.G) * (a.D + 1)) * sizeof(float) <= 60 * 1024;
}

void launch_window_write(const WindowArgs& a, const void* q, int64_t ldq, const void* k, int64_t ldk, const void* v,
                         int64_t ldv, const float* qw, const float* kw, float eps, int norm_all, void* q_out,
                         hipStream_t st) {
  if (a.T <= 0) return;
  const size_t lds = (size_t)((a.H + a.G) * a.D + a.H + a.G) * sizeof(float);
  hipLaunchKernelGGL(window_write_kernel, dim3(a.T), dim3(256), lds, st, a, q, ldq, k, ldk, v, ldv, qw, kw, eps, norm_all,
                     q_out);
}

void launch_window_pool(const WindowArgs& a, hipStream_t st) {
  if (a.T <= 0 || a.pool <= 0 || a.S <= 0) return;
  hipLaunchKernelGGL(window_pool_kernel, dim3(a.T), dim3(256), 0, st, a);
}

void launch_window_attn(const WindowArgs& a, const void* q, float scale, void* out, hipStream_t st) {
  if (a.T <= 0 || a.S <= 0) return;
  const int HC = heads_per_block(a);
  const int rep = a.H / a.G;
  hipLaunchKernelGGL(window_attn_kernel, dim3(a.T, a.G, (rep + HC - 1) / HC), dim3(256), window_attn_lds_bytes(a, HC), st,
                     a, q, HC, scale, out);
}

}  // namespace vgate
