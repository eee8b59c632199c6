// Generalized delta rule with per-channel decay, one fp32 state matrix S [key][value] per (sequence,
// head) kept in a state slot between steps:
//   w = exp(-c * sigmoid(wl + w0))        per key channel decay
//   a = sigmoid(al + ab)                  per key channel removal rate
//   u = k / sqrt(sum(k^2) + unit_eps)
//   S <- diag(w) S - (a * u) (u^T S) + k v^T        (both correction terms read the old S)
//   o  = S^T r;  out = o / rms(o) * nw * sigmoid(g)  (rms over the head)
// Three launches:
//   prep   (token, head) parallel: the per-channel fp32 vectors {w, a * u, k, r} and u of every token.
//   scan   the recurrence. Column v of S depends on no other column, so a head's D value columns are
//          split into slices of 8 and every (sequence, head, slice) is one wave: lane = (key group of
//          eight, column), D / 8 state entries in registers, the two sums over keys (u^T S, r^T S) are
//          D / 8 in-register FMAs + three cross-group lane exchanges: the per-token dependency chain of
//          a lone sequence's prefill is what bounds it, so the chain is kept short. Tokens are staged through LDS eight at
//          a time, the next eight loaded into registers while the current ones compute. A sequence's
//          tokens of the step run in order from the slot's state; a portion that starts at position 0
//          starts from zero, so a reused slot needs no clearing.
//   finish (token, head) parallel: head RMS norm, norm weight, output gate, store in the activation dtype.
#include "common.h"
#include "seq_launchers.h"

namespace vgate {
namespace {

__device__ __forceinline__ float ldx(const void* p, int64_t i, int f32) {
  return f32 ? reinterpret_cast<const float*>(p)[i] : bf2f(reinterpret_cast<const bf16_t*>(p)[i]);
}
__device__ __forceinline__ float sigm(float x) { return 1.f / (1.f + expf(-x)); }
// lane l gets lane l ^ 8's value: a rotation by 8 inside each row of 16 lanes (DPP row_ror:8), on the VALU
__device__ __forceinline__ float xor8(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xf, 0xf, false));
}

// one wave per (token, head): vec[t][h][d] = {w, a u, k, r}, un[t][h][d] = u
__global__ __launch_bounds__(64) void delta_prep_kernel(DeltaArgs p, int T, float4* __restrict__ vec,
                                                         float* __restrict__ un) {
  const int t = blockIdx.x, h = blockIdx.y;
  if (t >= p.query_start[p.S]) return;  // padding rows of a graph bucket
  const int D = p.D, lane = threadIdx.x;
  float kk[2], rr[2], aa[2], ww[2];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int d = lane + 64 * i;
    kk[i] = rr[i] = aa[i] = ww[i] = 0.f;
    if (d < D) {
      const int ch = h * D + d;
      const int64_t ix = (int64_t)t * p.ld + ch;
      kk[i] = ldx(p.k, ix, p.f32);
      rr[i] = ldx(p.r, ix, p.f32);
      aa[i] = sigm(ldx(p.a, ix, p.f32) + p.ab[ch]);
      ww[i] = expf(-p.decay_c * sigm(ldx(p.wl, (int64_t)t * p.ldw + ch, p.f32) + p.w0[ch]));
      ss = fmaf(kk[i], kk[i], ss);
    }
  }
  ss = wave_reduce_sum(ss);
  const float inv = 1.f / sqrtf(ss + p.unit_eps);
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int d = lane + 64 * i;
    if (d < D) {
      const float u = kk[i] * inv;
      const int64_t o = ((int64_t)t * p.H + h) * D + d;
      vec[o] = make_float4(ww[i], aa[i] * u, kk[i], rr[i]);
      un[o] = u;
    }
  }
}

constexpr int TC = 8;  // tokens staged per LDS buffer

// lane = 8 * q + c: key group q of 8 (keys [q DQ', (q + 1) DQ') with DQ' = ceil(D / 8)), value column c0 + c
template <int DQ>
__global__ __launch_bounds__(64) void delta_scan_kernel(DeltaArgs p, const float4* __restrict__ vec,
                                                         const float* __restrict__ un, float* __restrict__ oraw) {
  // quarter strides padded (DQ + 1 float4 / DQ + 4 floats): the four quarters' broadcast reads of one
  // instruction fall into different LDS banks. Entries of channels past D are zeroed once and never
  // written, so the token loops run DQ iterations with no bounds test (zeros leave S, u^T S and o alone).
  constexpr int QV = DQ + 1, QU = DQ + 4;
  __shared__ float4 lv[2][TC][8 * QV];
  __shared__ float lu[2][TC][8 * QU];
  __shared__ float lvv[2][TC][8];  // the slice's value columns of each staged token
  const int s = blockIdx.x, h = blockIdx.y, c0 = blockIdx.z * 8;
  const int slot = p.state_slots[s];
  const int t0 = p.query_start[s], t1 = p.query_start[s + 1];
  if (slot < 0 || t1 <= t0) return;
  const int D = p.D, lane = threadIdx.x;
  const int q = lane >> 3, c = c0 + (lane & 7);
  const int dq = (D + 7) >> 3;         // keys per group at run time (<= DQ)
  const int k0 = q * dq;
  const bool con = c < D;
  const int pos0 = p.context_lens[s] - (t1 - t0);
  float* sp = p.state + ((int64_t)slot * p.H + h) * D * D;
  float S[DQ];
#pragma unroll
  for (int j = 0; j < DQ; ++j)
    S[j] = (con && j < dq && k0 + j < D && pos0 > 0) ? sp[(int64_t)(k0 + j) * D + c] : 0.f;
  // staging: a token's D channels are D float4 + D floats; lane l moves channels l, l + 64 of each token
  float4 pv[TC][2];
  float pu[TC][2];
  float pvv;
  auto fetch = [&](int tb) {
#pragma unroll
    for (int i = 0; i < TC; ++i)
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const int d = lane + 64 * e, t = tb + i;
        const bool ok = d < D && t < t1;
        const int64_t o = ((int64_t)(ok ? t : t0) * p.H + h) * D + (ok ? d : 0);
        pv[i][e] = ok ? vec[o] : make_float4(0.f, 0.f, 0.f, 0.f);
        pu[i][e] = ok ? un[o] : 0.f;
      }
    {  // TC x 8 values, lane -> (token, column)
      const int t = tb + (lane >> 3), cc = c0 + (lane & 7);
      pvv = (t < t1 && cc < D) ? ldx(p.v, (int64_t)t * p.ld + h * D + cc, p.f32) : 0.f;
    }
  };
  // LDS index of channel d: quarter-major, padded to DQ per quarter
  auto put = [&](int buf) {
#pragma unroll
    for (int i = 0; i < TC; ++i)
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const int d = lane + 64 * e;
        if (d < D) {
          lv[buf][i][(d / dq) * QV + (d % dq)] = pv[i][e];
          lu[buf][i][(d / dq) * QU + (d % dq)] = pu[i][e];
        }
      }
    lvv[buf][lane >> 3][lane & 7] = pvv;
  };
  for (int e = lane; e < 2 * TC * 8 * QV; e += 64) (&lv[0][0][0])[e] = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int e = lane; e < 2 * TC * 8 * QU; e += 64) (&lu[0][0][0])[e] = 0.f;
  __syncthreads();
  fetch(t0);
  put(0);
  __syncthreads();
  int buf = 0;
  for (int tb = t0; tb < t1; tb += TC) {
    const bool more = tb + TC < t1;
    if (more) fetch(tb + TC);
    const int nt = min(TC, t1 - tb);
    // unrolled over the staged tokens, with token i + 1's vectors read from LDS into a second register
    // set before token i's FMAs and lane exchanges (they do not depend on the state)
    float4 xv[2][DQ];
    float xu[2][DQ], xvv[2];
    auto grab = [&](int i, int r) {
      const float4* tv = &lv[buf][i][q * QV];
      const float* tu = &lu[buf][i][q * QU];
#pragma unroll
      for (int j = 0; j < DQ; ++j) { xv[r][j] = tv[j]; xu[r][j] = tu[j]; }
      xvv[r] = lvv[buf][i][lane & 7];
    };
    grab(0, 0);
#pragma unroll
    for (int i = 0; i < TC; ++i) {
      if (i >= nt) break;
      if (i + 1 < TC) grab(i + 1, (i + 1) & 1);  // (past nt: stale but finite LDS, never used)
      const int r = i & 1;
      const float vv = xvv[r];
      float uS = 0.f;
#pragma unroll
      for (int j = 0; j < DQ; ++j) uS = fmaf(xu[r][j], S[j], uS);
      uS += xor8(uS);
      uS += xor16(uS);
      uS += xor32(uS);
      float o = 0.f;
#pragma unroll
      for (int j = 0; j < DQ; ++j) {
        const float4 x = xv[r][j];  // {w, a u, k, r}
        S[j] = fmaf(x.z, vv, fmaf(-x.y, uS, x.x * S[j]));
        o = fmaf(x.w, S[j], o);
      }
      o += xor8(o);
      o += xor16(o);
      o += xor32(o);
      if (con && q == 0) oraw[(int64_t)(tb + i) * p.H * D + h * D + c] = o;
    }
    if (more) {
      put(buf ^ 1);
      __syncthreads();
      buf ^= 1;
    }
  }
#pragma unroll
  for (int j = 0; j < DQ; ++j)
    if (con && j < dq && k0 + j < D) sp[(int64_t)(k0 + j) * D + c] = S[j];
}

// one wave per (token, head)
__global__ __launch_bounds__(64) void delta_finish_kernel(DeltaArgs p, const float* __restrict__ oraw) {
  const int t = blockIdx.x, h = blockIdx.y;
  if (t >= p.query_start[p.S]) return;
  const int D = p.D, lane = threadIdx.x;
  float o[2];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int d = lane + 64 * i;
    o[i] = d < D ? oraw[((int64_t)t * p.H + h) * D + d] : 0.f;
    ss = fmaf(o[i], o[i], ss);
  }
  ss = wave_reduce_sum(ss);
  const float inv = 1.f / sqrtf(ss / (float)D + p.eps);
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int d = lane + 64 * i;
    if (d < D) {
      const int ch = h * D + d;
      const float y = o[i] * inv * p.nw[ch] * sigm(ldx(p.g, (int64_t)t * p.ld + ch, p.f32));
      const int64_t oi = (int64_t)t * p.ldo + ch;
      if (p.f32) reinterpret_cast<float*>(p.out)[oi] = y;
      else reinterpret_cast<bf16_t*>(p.out)[oi] = f2bf(y);
    }
  }
}

}  // namespace

// scratch: T * H * D * 6 floats ({w, a u, k, r}, u, raw o)
void launch_delta_rule(const DeltaArgs& a, int T, float* scratch, hipStream_t st) {
  if (a.S <= 0 || a.H <= 0 || T <= 0) return;
  const int64_t n = (int64_t)T * a.H * a.D;
  float4* vec = reinterpret_cast<float4*>(scratch);
  float* un = scratch + 4 * n;
  float* oraw = scratch + 5 * n;
  hipLaunchKernelGGL(delta_prep_kernel, dim3(T, a.H), dim3(64), 0, st, a, T, vec, un);
  const dim3 grid(a.S, a.H, (a.D + 7) / 8);
  if (a.D <= 32) hipLaunchKernelGGL(delta_scan_kernel<4>, grid, dim3(64), 0, st, a, vec, un, oraw);
  else if (a.D <= 64) hipLaunchKernelGGL(delta_scan_kernel<8>, grid, dim3(64), 0, st, a, vec, un, oraw);
  else hipLaunchKernelGGL(delta_scan_kernel<16>, grid, dim3(64), 0, st, a, vec, un, oraw);
  hipLaunchKernelGGL(delta_finish_kernel, dim3(T, a.H), dim3(64), 0, st, a, oraw);
}

}  // namespace vgate
