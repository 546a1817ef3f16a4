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
// column per lane), and the dot products over D are finished through LDS.
//
// Tokens are taken in blocks of TB.  A block's k, q (and per-channel decays) are staged in LDS by the whole workgroup
// with coalesced loads, and the NEXT block is already in flight (in registers) while the current one is walked, so the
// dependent chain per token is LDS reads and FMAs, not a trip to memory.  The read-out's partial sums of a whole block
// are reduced at the block's end; only the delta rule needs a workgroup barrier per token (its S^T k sum crosses the
// waves).  A decode step is one block of one token: one pass over the state (read, update, write, coalesced along V).
// A sequence whose step starts at position 0 starts from S = 0; nothing is cleared when a slot changes hands.
#include "api_mixers.h"

namespace dsse {
namespace {

constexpr int kScanCols = 64;

template <int DPT, int TB, bool DELTA>
__global__ void matrix_scan_kernel(MatrixScanParams p, int R) {
  constexpr int E = TB * DPT / 64;  // staged elements of k (and q, a) per thread and block: TB * Dp / (64 R)
  extern __shared__ float lds[];
  const int seq = blockIdx.z, h = blockIdx.y;
  const int ql = p.q_len[seq];
  if (ql <= 0) return;
  const int tid = threadIdx.x, lane = tid & 63, r = tid >> 6;
  const int nthreads = R * 64;
  const int j = blockIdx.x * kScanCols + lane;
  const bool col_on = j < p.V;
  const int g = h / (p.H / p.G);
  const int D = p.D, Dp = R * DPT;
  const bool chan = p.decay_kind == 3;
  // LDS: k[2][TB][Dp] | q[2][TB][Dp] | (a[2][TB][Dp]) | sc[2][2][TB] (beta, scalar decay) | part[2][R][64] | opart[TB][R][64]
  float* ks = lds;
  float* qs = ks + 2 * TB * Dp;
  float* as = qs + 2 * TB * Dp;
  float* sc = as + (chan ? 2 * TB * Dp : 0);
  float* part_s = sc + 4 * TB;
  float* opart = part_s + 2 * R * kScanCols;
  const int row0 = p.q_start[seq];
  const bool fresh = p.ctx_len[seq] - ql == 0;
  float* st = p.state + (((int64_t)p.state_slot[seq] * p.H + h) * D) * p.V + j;
  float S[DPT];
#pragma unroll
  for (int i = 0; i < DPT; ++i) {
    const int d = r * DPT + i;
    S[i] = (!fresh && col_on && d < D) ? st[(int64_t)d * p.V] : 0.0f;
  }
  const float fixed = p.decay_kind == 1 ? p.decay[h] : 1.0f;
  float nk[E], nq[E], na[E], nv[TB], nsc0 = 0.f, nsc1 = 1.f;
  // request block b (tokens [b TB, b TB + TB)) into registers
  auto request = [&](int b) {
    const int t0 = b * TB;
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int idx = e * nthreads + tid;
      const int t = idx / Dp, d = idx - t * Dp;
      const bool on = t0 + t < ql && d < D;  // padded channels and tokens past the end are staged as k = q = 0, a = 1
      const int64_t row = row0 + t0 + t;
      nk[e] = on ? p.k[row * p.ldk + g * D + d] : 0.0f;
      nq[e] = on ? p.q[row * p.ldq + g * D + d] * p.q_scale : 0.0f;
      na[e] = (on && chan) ? p.decay[row * p.ldd + h * D + d] : 1.0f;
    }
#pragma unroll
    for (int t = 0; t < TB; ++t) nv[t] = (col_on && t0 + t < ql) ? p.v[(int64_t)(row0 + t0 + t) * p.ldv + h * p.V + j] : 0.0f;
    if (tid < TB && t0 + tid < ql) {
      const int64_t row = row0 + t0 + tid;
      nsc0 = DELTA ? p.beta[row * p.ldb + h] : 0.0f;
      nsc1 = p.decay_kind == 2 ? p.decay[row * p.ldd + h] : fixed;
    }
  };
  auto stage = [&](int buf) {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int idx = e * nthreads + tid;
      ks[buf * TB * Dp + idx] = nk[e];
      qs[buf * TB * Dp + idx] = nq[e];
      if (chan) as[buf * TB * Dp + idx] = na[e];
    }
    if (tid < TB) {
      sc[(buf * 2 + 0) * TB + tid] = nsc0;
      sc[(buf * 2 + 1) * TB + tid] = nsc1;
    }
  };
  const int nblocks = (ql + TB - 1) / TB;
  request(0);
  stage(0);
  for (int b = 0; b < nblocks; ++b) {
    const int buf = b & 1;
    float cv[TB];
#pragma unroll
    for (int t = 0; t < TB; ++t) cv[t] = nv[t];
    if (b + 1 < nblocks) request(b + 1);  // in flight while this block is walked
    __syncthreads();                      // this block's staging is visible; the previous block's opart has been read
    const int nt = ql - b * TB < TB ? ql - b * TB : TB;
#pragma unroll
    for (int t = 0; t < TB; ++t) {
      if (t < nt) {  // uniform
        const float* kb = ks + (buf * TB + t) * Dp + r * DPT;
        const float* qb = qs + (buf * TB + t) * Dp + r * DPT;
        if (chan) {
          const float* ab = as + (buf * TB + t) * Dp + r * DPT;
#pragma unroll
          for (int i = 0; i < DPT; ++i) S[i] *= ab[i];
        } else if (p.decay_kind != 0) {
          const float sa = sc[(buf * 2 + 1) * TB + t];
#pragma unroll
          for (int i = 0; i < DPT; ++i) S[i] *= sa;
        }
        float u = cv[t];
        if (DELTA) {
          float part = 0.f;
#pragma unroll
          for (int i = 0; i < DPT; ++i) part += S[i] * kb[i];
          if (R > 1) {  // two alternating strips: a strip is rewritten two tokens later, after a barrier in between
            float* ps = part_s + (t & 1) * R * kScanCols;
            ps[r * kScanCols + lane] = part;
            __syncthreads();
            part = 0.f;
            for (int w = 0; w < R; ++w) part += ps[w * kScanCols + lane];
          }
          u = sc[(buf * 2 + 0) * TB + t] * (cv[t] - part);
        }
        float o = 0.f;
#pragma unroll
        for (int i = 0; i < DPT; ++i) {
          S[i] += kb[i] * u;
          o += S[i] * qb[i];
        }
        opart[(t * R + r) * kScanCols + lane] = o;
      }
    }
    __syncthreads();  // the block's partial read-outs are complete; its staged inputs have been read
    // token t of the block is finished by wave t mod R
    for (int t = r; t < nt; t += R) {
      float o = 0.f;
      for (int w = 0; w < R; ++w) o += opart[(t * R + w) * kScanCols + lane];
      if (col_on) p.out[((int64_t)(row0 + b * TB + t) * p.H + h) * p.V + j] = o;
    }
    if (b + 1 < nblocks) stage(buf ^ 1);
  }
#pragma unroll
  for (int i = 0; i < DPT; ++i) {
    const int d = r * DPT + i;
    if (col_on && d < D) st[(int64_t)d * p.V] = S[i];
  }
}

template <int DPT, int TB>
hipError_t launch(const MatrixScanParams& p, hipStream_t st) {
  const int R = (p.D + DPT - 1) / DPT;
  const int Dp = R * DPT;
  dim3 grid((p.V + kScanCols - 1) / kScanCols, p.H, p.nseq);
  const size_t lds = (size_t)((p.decay_kind == 3 ? 6 : 4) * TB * Dp + 4 * TB + 2 * R * kScanCols + TB * R * kScanCols) *
                     sizeof(float);
  if (lds > 64 * 1024) return hipErrorInvalidValue;
  if (p.beta) hipLaunchKernelGGL((matrix_scan_kernel<DPT, TB, true>), grid, dim3(R * 64), lds, st, p, R);
  else hipLaunchKernelGGL((matrix_scan_kernel<DPT, TB, false>), grid, dim3(R * 64), lds, st, p, R);
  return hipGetLastError();
}

}  // namespace
}  // namespace dsse

extern "C" hipError_t dsse_matrix_scan(const dsse::MatrixScanParams* p, hipStream_t st) {
  if (p->nseq <= 0 || p->H <= 0) return hipSuccess;
  if (p->D < 1 || p->D > 512 || p->V < 1 || p->G < 1 || p->H % p->G) return hipErrorInvalidValue;
  // rows of S per lane and tokens per block: more waves shorten the per-token chain (up to 16 waves per workgroup),
  // the block is as long as 64 KB of LDS allow
  if (p->D <= 64) return dsse::launch<8, 8>(*p, st);
  if (p->D <= 128) return dsse::launch<16, 8>(*p, st);
  if (p->D <= 256) return dsse::launch<16, 4>(*p, st);
  return dsse::launch<32, 2>(*p, st);
}
