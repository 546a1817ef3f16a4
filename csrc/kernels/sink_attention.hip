// Causal softmax attention with a sink over paged keys and values of any head width (grouped key/value heads).
//
//   score_j = scale (q . k_j),  j in [max(0, pos - window + 1), pos]
//   out     = sum_j exp(score_j - m) v_j / (sum_j exp(score_j - m) + exp(sink_h - m)),  m = max(max_j score_j, sink_h)
//   out    *= sigmoid(gate[row, h])                                                      (optional)
//
// The sink is a learned logit with no key and no value: it only enlarges the denominator, so a head can attend to
// "nothing".  Scores, the running maximum, the weights and the output sums are fp32 in both element types; queries
// arrive in fp32 (normed and rotated), keys and values are read from their pages in the cache's element type.
//
// Row kernel: a workgroup serves `qt` query rows of one head; for each row its four waves split the keys in chunks of
// 64 (one key per lane for the scores, then one output coordinate per lane and 64 broadcast weights for the values),
// keep their own running (max, sum, output) and are merged through LDS.  A decode row and a prompt row take the same
// path, so a position's result does not depend on how the prompt was cut.
#include "api_mixers.h"

namespace dsse {
namespace {

constexpr int kMaxV = 512;
constexpr int kAccs = kMaxV / 64;

// q (LDS, fp32) . key row (global): 16-byte loads when the row width allows
DEV float dot_row(const float* q, const bf16* k, int D) {
  float s = 0.f;
  int d = 0;
  if (D % 8 == 0) {
    for (; d < D; d += 8) {
      const bf16x8 kv = *reinterpret_cast<const bf16x8*>(k + d);
#pragma unroll
      for (int e = 0; e < 8; ++e) s += q[d + e] * (float)kv[e];
    }
  }
  for (; d < D; ++d) s += q[d] * (float)k[d];
  return s;
}
DEV float dot_row(const float* q, const float* k, int D) {
  float s = 0.f;
  int d = 0;
  if (D % 4 == 0) {
    for (; d < D; d += 4) {
      const f32x4 kv = *reinterpret_cast<const f32x4*>(k + d);
#pragma unroll
      for (int e = 0; e < 4; ++e) s += q[d + e] * kv[e];
    }
  }
  for (; d < D; ++d) s += q[d] * k[d];
  return s;
}

template <typename T>
__global__ __launch_bounds__(256) void sink_attention_kernel(SinkAttnParams p) {
  __shared__ float qs[512];
  __shared__ float m_s[4], l_s[4];
  __shared__ float acc_s[4][kMaxV];
  const int work = blockIdx.x, h = blockIdx.y;
  const int seq = p.work_seq[work], tile = p.work_tile[work];
  const int ql = p.q_len[seq];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int g = h / (p.H / p.G);
  const int D = p.D, V = p.V;
  const int* bt = p.block_tables + (int64_t)seq * p.max_blocks;
  const T* kc = reinterpret_cast<const T*>(p.k);
  const T* vc = reinterpret_cast<const T*>(p.v);
  const float sink = p.sink ? p.sink[h] : -INFINITY;
  for (int i = 0; i < p.qt; ++i) {
    const int off = tile * p.qt + i;
    if (off >= ql) break;  // uniform for the workgroup
    const int row = p.q_start[seq] + off;
    const int pos = p.ctx_len[seq] - ql + off;
    const int lo = pos - p.window + 1 > 0 ? pos - p.window + 1 : 0;
    const int nkeys = pos - lo + 1;
    __syncthreads();  // the previous row's merge has read qs / acc_s
    for (int d = threadIdx.x; d < D; d += blockDim.x) qs[d] = p.q[((int64_t)row * p.H + h) * D + d];
    __syncthreads();
    float m = -INFINITY, l = 0.f;
    float acc[kAccs];
#pragma unroll
    for (int a = 0; a < kAccs; ++a) acc[a] = 0.f;
    for (int c = wave; c * 64 < nkeys; c += 4) {
      const int jj = c * 64 + lane;
      const bool on = jj < nkeys;
      const int j = lo + (on ? jj : 0);
      int page = bt[j / kBS];
      page = (unsigned)page < (unsigned)p.num_blocks ? page : 0;
      const int krow = (page * kBS + j % kBS) * p.G + g;
      const float s_dot = dot_row(qs, kc + (int64_t)krow * D, D);
      float s = s_dot;
      s = on ? s * p.scale : -INFINITY;
      const float m_new = fmaxf(m, wave_max(s));  // finite: the chunk holds at least one key
      const float w = on ? expf(s - m_new) : 0.f;
      const float f = expf(m - m_new);            // 0 when m was -inf
      l = l * f + wave_sum(w);
      m = m_new;
#pragma unroll
      for (int a = 0; a < kAccs; ++a) acc[a] *= f;
      const int cnt = nkeys - c * 64 < 64 ? nkeys - c * 64 : 64;
      for (int t = 0; t < cnt; ++t) {
        const float wt = __shfl(w, t);
        const int vrow = __shfl(krow, t);
        const T* vp = vc + (int64_t)vrow * V;
#pragma unroll
        for (int a = 0; a < kAccs; ++a)
          if (a * 64 + lane < V) acc[a] += wt * (float)vp[a * 64 + lane];
      }
    }
    if (lane == 0) {
      m_s[wave] = m;
      l_s[wave] = l;
    }
#pragma unroll
    for (int a = 0; a < kAccs; ++a)
      if (a * 64 + lane < V) acc_s[wave][a * 64 + lane] = acc[a];
    __syncthreads();
    float mm = sink;
    for (int w = 0; w < 4; ++w) mm = fmaxf(mm, m_s[w]);
    float den = p.sink ? expf(sink - mm) : 0.f;
    float fw[4];
    for (int w = 0; w < 4; ++w) {
      fw[w] = m_s[w] == -INFINITY ? 0.f : expf(m_s[w] - mm);
      den += l_s[w] * fw[w];
    }
    const float gate = p.gate ? 1.0f / (1.0f + expf(-p.gate[(int64_t)row * p.ldg + h])) : 1.0f;
    T* out = reinterpret_cast<T*>(p.out) + ((int64_t)row * p.H + h) * V;
    for (int d = threadIdx.x; d < V; d += blockDim.x) {
      float o = 0.f;
      for (int w = 0; w < 4; ++w) o += acc_s[w][d] * fw[w];
      out[d] = (T)(o / den * gate);
    }
  }
}

}  // namespace
}  // namespace dsse

extern "C" hipError_t dsse_sink_attention(int num_work, const dsse::SinkAttnParams* p, hipStream_t st) {
  if (num_work <= 0 || p->H <= 0) return hipSuccess;
  if (p->D > 512 || p->V > dsse::kMaxV || p->H % p->G) return hipErrorInvalidValue;
  dim3 grid(num_work, p->H);
  if (p->f32) hipLaunchKernelGGL(dsse::sink_attention_kernel<float>, grid, dim3(256), 0, st, *p);
  else hipLaunchKernelGGL(dsse::sink_attention_kernel<bf16>, grid, dim3(256), 0, st, *p);
  return hipGetLastError();
}
