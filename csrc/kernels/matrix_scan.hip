// Matrix-state recurrences over the engine's per-sequence state slots: per (sequence, head) a state S [D, V] in fp32
// that each token updates and reads,
//
//     S = a S                       a: nothing, one number per head, one per (token, head), or one per (token, head,
//                                      key channel) -- fixed-decay retention, gated delta rule, gated linear attention
//     u = beta (v - S^T k)          with beta (the delta rule: the write corrects what the key already recalls),
//     u = v                         without
//     S = S + k u^T
//     o = S^T (q_scale q)           the read-out sees the current token's write
//
// Column j of S evolves independently of the other columns, so the work is laid out by columns: a workgroup owns 64
// columns of one (sequence, head); wave r of it holds rows [r DPT, (r + 1) DPT) of those columns in registers (one
// column per lane), and the two dot products over D are finished through LDS.  The token's k, q (and per-channel
// decay) are staged in LDS once per workgroup; the next token's are requested from global memory before the current
// token's math, so a prompt portion costs one short dependent chain per token and a decode step is one pass over the
// state (read, update, write: coalesced along V).  A sequence whose step starts at position 0 starts from S = 0;
// nothing is cleared when a slot changes hands.
#include "api_mixers.h"

namespace dsse {
namespace {

constexpr int kScanCols = 64;

template <int DPT, bool DELTA>
__global__ void matrix_scan_kernel(MatrixScanParams p, int R) {
  extern __shared__ float lds[];
  const int seq = blockIdx.z, h = blockIdx.y;
  const int ql = p.q_len[seq];
  if (ql <= 0) return;
  const int lane = threadIdx.x & 63, r = threadIdx.x >> 6;
  const int j = blockIdx.x * kScanCols + lane;
  const bool col_on = j < p.V;
  const int g = h / (p.H / p.G);
  const int D = p.D, Dp = R * DPT;
  // LDS: k[2][Dp] | q[2][Dp] | a[2][Dp] | red[2][R][64] | red2[2][R][64]
  float* ks = lds;
  float* qs = ks + 2 * Dp;
  float* as = qs + 2 * Dp;
  float* red = as + 2 * Dp;
  float* red2 = red + 2 * R * kScanCols;
  const int row0 = p.q_start[seq];
  const bool fresh = p.ctx_len[seq] - ql == 0;
  float* st = p.state + (((int64_t)p.state_slot[seq] * p.H + h) * D) * p.V + j;
  float S[DPT];
#pragma unroll
  for (int i = 0; i < DPT; ++i) {
    const int d = r * DPT + i;
    S[i] = (!fresh && col_on && d < D) ? st[(int64_t)d * p.V] : 0.0f;
  }
  const int tid = threadIdx.x;
  const bool ld_on = tid < Dp;           // this thread stages element tid of k, q (and the per-channel decay)
  const bool ld_real = tid < D;          // padded rows (d >= D) are staged as zeros: they leave S at zero
  float nk = 0.f, nq = 0.f, na = 1.f, nv = 0.f, nb = 0.f, nsa = 1.f;
  auto request = [&](int t) {
    const int64_t row = row0 + t;
    if (ld_real) {
      nk = p.k[row * p.ldk + g * D + tid];
      nq = p.q[row * p.ldq + g * D + tid] * p.q_scale;
      if (p.decay_kind == 3) na = p.decay[row * p.ldd + h * D + tid];
    }
    nv = col_on ? p.v[row * p.ldv + h * p.V + j] : 0.0f;
    if (DELTA) nb = p.beta[row * p.ldb + h];
    if (p.decay_kind == 2) nsa = p.decay[row * p.ldd + h];
  };
  if (p.decay_kind == 1) nsa = p.decay[h];
  request(0);
  for (int t = 0; t < ql; ++t) {
    const int buf = t & 1;
    if (ld_on) {
      ks[buf * Dp + tid] = nk;
      qs[buf * Dp + tid] = nq;
      as[buf * Dp + tid] = na;
    }
    const float vj = nv, beta = nb, sa = nsa;
    if (t + 1 < ql) request(t + 1);  // in flight during this token's math
    __syncthreads();
    const float* kb = ks + buf * Dp + r * DPT;
    const float* qb = qs + buf * Dp + r * DPT;
    const float* ab = as + buf * Dp + r * DPT;
    if (p.decay_kind == 3) {
#pragma unroll
      for (int i = 0; i < DPT; ++i) S[i] *= ab[i];
    } else if (p.decay_kind != 0) {
#pragma unroll
      for (int i = 0; i < DPT; ++i) S[i] *= sa;
    }
    float u = vj;
    if (DELTA) {
      float part = 0.f;
#pragma unroll
      for (int i = 0; i < DPT; ++i) part += S[i] * kb[i];
      if (R > 1) {
        red[(buf * R + r) * kScanCols + lane] = part;
        __syncthreads();
        part = 0.f;
        for (int w = 0; w < R; ++w) part += red[(buf * R + w) * kScanCols + lane];
      }
      u = beta * (vj - part);
    }
    float o = 0.f;
#pragma unroll
    for (int i = 0; i < DPT; ++i) {
      S[i] += kb[i] * u;
      o += S[i] * qb[i];
    }
    if (R > 1) {
      red2[(buf * R + r) * kScanCols + lane] = o;
      __syncthreads();
      if (r == 0) {
        o = 0.f;
        for (int w = 0; w < R; ++w) o += red2[(buf * R + w) * kScanCols + lane];
      }
    }
    if (r == 0 && col_on) p.out[((int64_t)(row0 + t) * p.H + h) * p.V + j] = o;
  }
#pragma unroll
  for (int i = 0; i < DPT; ++i) {
    const int d = r * DPT + i;
    if (col_on && d < D) st[(int64_t)d * p.V] = S[i];
  }
}

template <int DPT>
hipError_t launch(const MatrixScanParams& p, hipStream_t st) {
  const int R = (p.D + DPT - 1) / DPT;
  dim3 grid((p.V + kScanCols - 1) / kScanCols, p.H, p.nseq);
  const size_t lds = (size_t)(6 * R * DPT + 4 * R * kScanCols) * sizeof(float);
  if (p.beta) hipLaunchKernelGGL((matrix_scan_kernel<DPT, true>), grid, dim3(R * 64), lds, st, p, R);
  else hipLaunchKernelGGL((matrix_scan_kernel<DPT, false>), grid, dim3(R * 64), lds, st, p, R);
  return hipGetLastError();
}

}  // namespace
}  // namespace dsse

extern "C" hipError_t dsse_matrix_scan(const dsse::MatrixScanParams* p, hipStream_t st) {
  if (p->nseq <= 0 || p->H <= 0) return hipSuccess;
  if (p->D < 1 || p->D > 512 || p->V < 1 || p->G < 1 || p->H % p->G) return hipErrorInvalidValue;
  // rows of S per lane: more waves shorten the per-token chain, up to 16 waves (1024 threads) per workgroup
  if (p->D <= 64) return dsse::launch<8>(*p, st);
  if (p->D <= 256) return dsse::launch<16>(*p, st);
  return dsse::launch<32>(*p, st);
}
