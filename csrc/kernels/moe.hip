// Routed mixture of experts: router (fp32 logits, top-k, softmax over the chosen logits only) and the token-major
// expert feed-forward (each row walks its chosen experts and the always-on shared expert).
//
//   moe_router   one wave per row: logits z[e] = w[e] . x + b[e] in fp32 (lanes split the width, wave reduction), then
//                the `top` largest (lowest index first among equals) and their softmax.
//   moe_ffn      one workgroup per row: x in LDS; per expert, a wave per hidden unit computes silu(gate . x) * (up . x)
//                into LDS, then a wave per output coordinate adds weight * (down . hidden).  The row's result leaves as
//                fp32 (the residual norm follows).  Each expert's weights are read once per row that chose it: the
//                decode-shaped path (few rows per expert), and correct for any row count.
#include "api_layers.h"

namespace dsse {
namespace {

template <typename T>
__global__ __launch_bounds__(64) void moe_router_kernel(MoeRouterParams p) {
  extern __shared__ float z[];  // [E]
  const int row = blockIdx.x, lane = threadIdx.x;
  const T* x = reinterpret_cast<const T*>(p.x) + (int64_t)row * p.W;
  const T* w = reinterpret_cast<const T*>(p.w);
  for (int e = 0; e < p.E; ++e) {
    float s = 0.f;
    for (int d = lane; d < p.W; d += 64) s += (float)w[(int64_t)e * p.W + d] * (float)x[d];
    s = wave_sum(s);
    if (lane == 0) z[e] = s + (p.b ? (float)reinterpret_cast<const T*>(p.b)[e] : 0.0f);
  }
  __syncthreads();
  if (lane == 0) {
    int* idx = p.topk_idx + (int64_t)row * p.top;
    float* wt = p.topk_w + (int64_t)row * p.top;
    float mx = 0.f;
    for (int k = 0; k < p.top; ++k) {
      int best = -1;
      float bv = 0.f;
      for (int e = 0; e < p.E; ++e) {
        bool used = false;
        for (int j = 0; j < k; ++j) used |= idx[j] == e;
        if (used) continue;
        if (best < 0 || z[e] > bv) best = e, bv = z[e];  // a NaN logit (an inactive row's garbage) still picks e
      }
      idx[k] = best < 0 ? 0 : best;
      wt[k] = bv;
      if (k == 0) mx = bv;
    }
    float sum = 0.f;
    for (int k = 0; k < p.top; ++k) {
      wt[k] = expf(wt[k] - mx);
      sum += wt[k];
    }
    for (int k = 0; k < p.top; ++k) wt[k] /= sum;
  }
}

template <typename T>
DEV void expert_row(const T* gate, const T* up, const T* down, int W, int F, float wgt, const float* xs, float* hs,
                    float* acc) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  for (int f = wave; f < F; f += nw) {
    float g = 0.f, u = 0.f;
    const T* gr = gate + (int64_t)f * W;
    const T* ur = up + (int64_t)f * W;
    for (int d = lane; d < W; d += 64) {
      const float xv = xs[d];
      g += (float)gr[d] * xv;
      u += (float)ur[d] * xv;
    }
    g = wave_sum(g);
    u = wave_sum(u);
    if (lane == 0) hs[f] = g / (1.0f + expf(-g)) * u;
  }
  __syncthreads();
  for (int d = wave; d < W; d += nw) {
    float s = 0.f;
    const T* dr = down + (int64_t)d * F;
    for (int f = lane; f < F; f += 64) s += (float)dr[f] * hs[f];
    s = wave_sum(s);
    if (lane == 0) acc[d] += wgt * s;
  }
  __syncthreads();
}

template <typename T>
__global__ __launch_bounds__(256) void moe_ffn_kernel(MoeFfnParams p) {
  extern __shared__ float smem[];
  float* xs = smem;            // [W]
  float* acc = smem + p.W;     // [W]
  float* hs = acc + p.W;       // [max(F, Fs)]
  const int row = blockIdx.x;
  const T* x = reinterpret_cast<const T*>(p.x) + (int64_t)row * p.W;
  for (int d = threadIdx.x; d < p.W; d += blockDim.x) {
    xs[d] = (float)x[d];
    acc[d] = 0.f;
  }
  __syncthreads();
  for (int k = 0; k < p.top; ++k) {
    int e = p.topk_idx[(int64_t)row * p.top + k];
    e = (unsigned)e < (unsigned)p.E ? e : 0;
    const float wgt = p.topk_w[(int64_t)row * p.top + k];
    expert_row<T>(reinterpret_cast<const T*>(p.gate) + (int64_t)e * p.F * p.W,
                  reinterpret_cast<const T*>(p.up) + (int64_t)e * p.F * p.W,
                  reinterpret_cast<const T*>(p.down) + (int64_t)e * p.W * p.F, p.W, p.F, wgt, xs, hs, acc);
  }
  if (p.sgate)
    expert_row<T>(reinterpret_cast<const T*>(p.sgate), reinterpret_cast<const T*>(p.sup),
                  reinterpret_cast<const T*>(p.sdown), p.W, p.Fs, 1.0f, xs, hs, acc);
  for (int d = threadIdx.x; d < p.W; d += blockDim.x) p.out[(int64_t)row * p.W + d] = acc[d];
}

}  // namespace
}  // namespace dsse

extern "C" hipError_t dsse_moe_router(const dsse::MoeRouterParams* p, hipStream_t st) {
  if (p->M <= 0) return hipSuccess;
  const size_t lds = sizeof(float) * p->E;
  if (p->f32) hipLaunchKernelGGL(dsse::moe_router_kernel<float>, dim3(p->M), dim3(64), lds, st, *p);
  else hipLaunchKernelGGL(dsse::moe_router_kernel<bf16>, dim3(p->M), dim3(64), lds, st, *p);
  return hipGetLastError();
}

extern "C" hipError_t dsse_moe_ffn(const dsse::MoeFfnParams* p, hipStream_t st) {
  if (p->M <= 0) return hipSuccess;
  const int fmax = p->F > p->Fs ? p->F : p->Fs;
  const size_t lds = sizeof(float) * (2 * (size_t)p->W + fmax);
  if (lds > 64 * 1024) return hipErrorInvalidValue;
  if (p->f32) hipLaunchKernelGGL(dsse::moe_ffn_kernel<float>, dim3(p->M), dim3(256), lds, st, *p);
  else hipLaunchKernelGGL(dsse::moe_ffn_kernel<bf16>, dim3(p->M), dim3(256), lds, st, *p);
  return hipGetLastError();
}
