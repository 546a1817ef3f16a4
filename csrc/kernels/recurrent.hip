// Gated linear recurrence with a short causal convolution in front (the recurrent block of Griffin-style designs), over
// the engine's per-sequence state slots.
//
//   conv_state   out[t, c] = b[c] + sum_k taps[c, k] * in[t - (K - 1) + k, c]; inputs before the step's first row come
//                from the slot's tail (the last K - 1 inputs of the sequence), zeros before the sequence's start.  The
//                tail is rewritten with the step's last K - 1 inputs (shifted in place when the step is shorter).
//   lru_scan     r = sigmoid(gate_r), i = sigmoid(gate_i), log a = -c r softplus(lam), S = a S + sqrt(1 - a^2) i u,
//                out = S * y.  The state S is fp32 and lives in the sequence's slot; a sequence's first step starts from
//                S = 0 (position 0 is not special-cased beyond that: the recurrence's own formula applies to it).
//
// One thread per (sequence, channel), the step's rows in order: a decode step is one iteration, a prompt portion is a
// loop over its rows.  Everything here is fp32 whatever the element type of the projections around it.
#include "api_layers.h"

namespace dsse {
namespace {

DEV float sigmoidf(float x) { return 1.0f / (1.0f + expf(-x)); }
DEV float softplusf(float x) { return x > 20.0f ? x : log1pf(expf(x)); }

template <typename T>
__global__ __launch_bounds__(256) void conv_state_kernel(ConvStateParams p) {
  const int seq = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int ql = p.q_len[seq];
  if (c >= p.C || ql <= 0) return;
  const int K = p.K, Kt = K - 1;
  const int row0 = p.q_start[seq];
  const bool fresh = p.ctx_len[seq] - ql == 0;  // the sequence starts in this step: nothing before it
  float* tail = p.tail + (int64_t)p.state_slot[seq] * Kt * p.C + c;  // tail[j * C]: input at offset j - Kt
  const T* taps = reinterpret_cast<const T*>(p.taps) + (int64_t)c * K;
  const float bias = p.bias ? (float)reinterpret_cast<const T*>(p.bias)[c] : 0.0f;
  const float* in = p.in + (int64_t)row0 * p.C + c;
  for (int t = 0; t < ql; ++t) {
    float v = bias;
    for (int k = 0; k < K; ++k) {
      const int i = t - Kt + k;
      const float x = i >= 0 ? in[(int64_t)i * p.C] : (fresh ? 0.0f : tail[(int64_t)(Kt + i) * p.C]);
      v += (float)taps[k] * x;
    }
    p.out[(int64_t)(row0 + t) * p.C + c] = v;
    reinterpret_cast<T*>(p.out_b)[(int64_t)(row0 + t) * p.C + c] = (T)v;
  }
  // new tail, ascending: entry j takes the input at offset ql - Kt + j, which for a short step is the old entry
  // j + ql (> j, not yet overwritten)
  for (int j = 0; j < Kt; ++j) {
    const int i = ql - Kt + j;
    tail[(int64_t)j * p.C] = i >= 0 ? in[(int64_t)i * p.C] : (fresh ? 0.0f : tail[(int64_t)(Kt + i) * p.C]);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void lru_scan_kernel(LruScanParams p) {
  const int seq = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int ql = p.q_len[seq];
  if (c >= p.C || ql <= 0) return;
  const int row0 = p.q_start[seq];
  float* st = p.state + (int64_t)p.state_slot[seq] * p.C + c;
  float S = p.ctx_len[seq] - ql == 0 ? 0.0f : *st;
  const float sp = softplusf((float)reinterpret_cast<const T*>(p.lam)[c]);
  const int b = c / p.bw, o = c % p.bw;
  const T* y = reinterpret_cast<const T*>(p.y);
  T* out = reinterpret_cast<T*>(p.out);
  for (int t = 0; t < ql; ++t) {
    const int64_t row = row0 + t;
    const float* g = p.gates + row * 2 * p.C + (int64_t)b * 2 * p.bw;
    const float r = sigmoidf(g[o]), gi = sigmoidf(g[p.bw + o]);
    const float log_a = -p.c * r * sp;
    const float a = expf(log_a);
    const float mult = sqrtf(-expm1f(2.0f * log_a));  // sqrt(1 - a^2) without the cancellation near a = 1
    S = a * S + mult * gi * p.u[row * p.C + c];
    out[row * p.C + c] = (T)(S * (float)y[row * p.C + c]);
  }
  *st = S;
}

}  // namespace
}  // namespace dsse

extern "C" hipError_t dsse_conv_state(const dsse::ConvStateParams* p, hipStream_t st) {
  if (p->nseq <= 0) return hipSuccess;
  dim3 grid((p->C + 255) / 256, p->nseq);
  if (p->f32) hipLaunchKernelGGL(dsse::conv_state_kernel<float>, grid, dim3(256), 0, st, *p);
  else hipLaunchKernelGGL(dsse::conv_state_kernel<bf16>, grid, dim3(256), 0, st, *p);
  return hipGetLastError();
}

extern "C" hipError_t dsse_lru_scan(const dsse::LruScanParams* p, hipStream_t st) {
  if (p->nseq <= 0) return hipSuccess;
  dim3 grid((p->C + 255) / 256, p->nseq);
  if (p->f32) hipLaunchKernelGGL(dsse::lru_scan_kernel<float>, grid, dim3(256), 0, st, *p);
  else hipLaunchKernelGGL(dsse::lru_scan_kernel<bf16>, grid, dim3(256), 0, st, *p);
  return hipGetLastError();
}
