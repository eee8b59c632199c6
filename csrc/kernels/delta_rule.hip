// Generalized delta rule with per-channel decay, one fp32 state matrix S [key][value] per (sequence,
// head) kept in a state slot between steps:
//   w = exp(-c * sigmoid(wl + w0))        per key channel decay
//   a = sigmoid(al + ab)                  per key channel removal rate
//   u = k / sqrt(sum(k^2) + unit_eps)
//   S <- diag(w) S - (a * u) (u^T S) + k v^T        (both correction terms read the old S)
//   o  = S^T r;  out = o / rms(o) * nw * sigmoid(g)  (rms over the head)
// One workgroup per (sequence, head), thread v owns column v of S in registers; the token's per-channel
// vectors are shared through LDS. A sequence's tokens of the step (a prompt portion or one decoded
// token) run in order from the slot's state; a portion that starts at position 0 starts from zero, so
// a reused slot needs no clearing. The next token's inputs are loaded while the current one computes.
#include "common.h"
#include "seq_launchers.h"

namespace vgate {
namespace {

__device__ __forceinline__ float ldx(const void* p, int64_t i, int f32) {
  return f32 ? reinterpret_cast<const float*>(p)[i] : bf2f(reinterpret_cast<const bf16_t*>(p)[i]);
}
__device__ __forceinline__ float sigm(float x) { return 1.f / (1.f + expf(-x)); }

struct TokIn { float r, k, v, g, a, wl; };

__device__ __forceinline__ TokIn load_tok(const DeltaArgs& p, int64_t t, int c, bool on) {
  TokIn x{0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (on) {
    const int64_t i = t * p.ld + c;
    x.r = ldx(p.r, i, p.f32); x.k = ldx(p.k, i, p.f32); x.v = ldx(p.v, i, p.f32);
    x.g = ldx(p.g, i, p.f32); x.a = ldx(p.a, i, p.f32);
    x.wl = ldx(p.wl, t * p.ldw + c, p.f32);
  }
  return x;
}

template <int DMAX>
__global__ __launch_bounds__(DMAX) void delta_rule_kernel(DeltaArgs p) {
  __shared__ float4 tok[DMAX];  // {w, a * u, k, r} per key channel
  __shared__ float us[DMAX];
  __shared__ float red[16];
  const int s = blockIdx.x, h = blockIdx.y;
  const int slot = p.state_slots[s];
  const int t0 = p.query_start[s], t1 = p.query_start[s + 1];
  if (slot < 0 || t1 <= t0) return;
  const int D = p.D;
  const int v = threadIdx.x;
  const bool on = v < D;
  const int ch = h * D + v;
  const int pos0 = p.context_lens[s] - (t1 - t0);
  float* sp = p.state + ((int64_t)slot * p.H + h) * D * D;
  float S[DMAX];
#pragma unroll
  for (int k = 0; k < DMAX; ++k) S[k] = (on && k < D && pos0 > 0) ? sp[(int64_t)k * D + v] : 0.f;
  const float w0 = on ? p.w0[ch] : 0.f, ab = on ? p.ab[ch] : 0.f, nw = on ? p.nw[ch] : 0.f;
  TokIn cur = load_tok(p, t0, ch, on);
  for (int t = t0; t < t1; ++t) {
    const TokIn nxt = load_tok(p, t + 1, ch, on && t + 1 < t1);
    const float ksum = block_reduce_sum(cur.k * cur.k, red);
    const float u = cur.k * (1.f / sqrtf(ksum + p.unit_eps));
    const float w = expf(-p.decay_c * sigm(cur.wl + w0));
    const float a = sigm(cur.a + ab);
    if (on) {
      tok[v] = make_float4(w, a * u, cur.k, cur.r);
      us[v] = u;
    }
    __syncthreads();
    float uS = 0.f;
#pragma unroll
    for (int k = 0; k < DMAX; ++k)
      if (k < D) uS = fmaf(us[k], S[k], uS);
    float o = 0.f;
#pragma unroll
    for (int k = 0; k < DMAX; ++k)
      if (k < D) {
        const float4 c = tok[k];
        S[k] = fmaf(c.z, cur.v, fmaf(-c.y, uS, c.x * S[k]));
        o = fmaf(c.w, S[k], o);
      }
    if (!on) o = 0.f;
    const float ss = block_reduce_sum(o * o, red);  // (its barriers also fence this token's LDS reads)
    if (on) {
      const float y = o * (1.f / sqrtf(ss / (float)D + p.eps)) * nw * sigm(cur.g);
      const int64_t oi = (int64_t)t * p.ldo + ch;
      if (p.f32) reinterpret_cast<float*>(p.out)[oi] = y;
      else reinterpret_cast<bf16_t*>(p.out)[oi] = f2bf(y);
    }
    cur = nxt;
  }
  if (on) {
#pragma unroll
    for (int k = 0; k < DMAX; ++k)
      if (k < D) sp[(int64_t)k * D + v] = S[k];
  }
}

}  // namespace

void launch_delta_rule(const DeltaArgs& a, hipStream_t st) {
  if (a.S <= 0 || a.H <= 0) return;
  const dim3 grid(a.S, a.H);
  if (a.D <= 64) hipLaunchKernelGGL(delta_rule_kernel<64>, grid, dim3(64), 0, st, a);
  else hipLaunchKernelGGL(delta_rule_kernel<128>, grid, dim3(128), 0, st, a);
}

}  // namespace vgate
