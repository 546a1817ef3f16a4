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
// Two kernels: this one for decode-sized steps (a row or two per sequence: what counts is the state traffic) and the
// wave-local one further down for prompt portions (what counts is the chain per token).
//
// Column j of S evolves independently of the other columns, so the work is laid out by columns: a workgroup owns 16
// columns of one (sequence, head).  Lane (c, dg) of wave r holds DPT rows of column c -- rows (4 r + dg) DPT + i -- in
// registers, so a dot product over D is DPT FMAs per lane, a sum over the wave's four 16-lane rows (two row swaps, no
// LDS) and a short sum over the waves through LDS.  A small DPT spreads one head's state over many waves, so a decode
// step's pass over the state (read, update, write) is wide; a state entry is kept tile-major (below) so that the pass
// moves whole lines.
//
// Tokens are taken in blocks of TB (a decode step is one block of one token; a step with two or three rows per
// sequence walks them here too).  A block's k, q (and per-channel decays) are staged in LDS by the whole workgroup with
// coalesced loads, the NEXT block is already in flight (in registers) while the current one is walked, the read-out's
// partial sums of a block are reduced at the block's end, and the delta rule needs one workgroup barrier per token
// (its S^T k sum crosses the waves).  A sequence whose step starts at position 0 starts from S = 0; nothing is cleared
// when a slot changes hands.
#include "api_mixers.h"

namespace dsse {
namespace {

constexpr int kScanCols = 16;

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every outstanding global load, which
// would land the next block's prefetch at each barrier; here those loads stay in flight until stage() uses them (the
// compiler's own vmcnt wait at the first use of their registers).
DEV void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

template <int DPT, int TB, bool DELTA>
__global__ __launch_bounds__(1024) void matrix_scan_kernel(MatrixScanParams p, int R) {
  constexpr int RW = 4 * DPT;        // rows of S per wave
  constexpr int E = TB * RW / 64;    // staged elements of k (and q, a) per thread and block: TB * Dp / (64 R)
  static_assert(E >= 1 && E * 64 == TB * RW, "a block's staging divides evenly over the workgroup");
  extern __shared__ __align__(16) float lds[];
  const int seq = blockIdx.z, h = blockIdx.y;
  const int ql = p.q_len[seq];
  if (ql <= 0) return;
  const int tid = threadIdx.x, lane = tid & 63, r = tid >> 6;
  const int c = lane & 15, dg = lane >> 4;
  const int nthreads = R * 64;
  const int j = blockIdx.x * kScanCols + c;
  const bool col_on = j < p.V;
  const int g = h / (p.H / p.G);
  const int D = p.D, Dp = R * RW;
  const int d0 = (4 * r + dg) * DPT;  // this lane's first row
  const bool chan = p.decay_kind == 3;
  // LDS: k[2][TB][Dp] | q[2][TB][Dp] | (a[2][TB][Dp]) | sc[2][2][TB] (beta, scalar decay) | part[2][R][16] | opart[TB][R][16]
  float* ks = lds;
  float* qs = ks + 2 * TB * Dp;
  float* as = qs + 2 * TB * Dp;
  float* sc = as + (chan ? 2 * TB * Dp : 0);
  float* part_s = sc + 4 * TB;
  float* opart = part_s + 2 * R * kScanCols;
  const int row0 = p.q_start[seq];
  // where the walk starts from and where its end state goes: the sequence's slot (zeros at position 0), or, for a
  // chunk of the two-level walk, the entries its lists name
  // State entries [H, D, V] are kept tile-major when V is a multiple of 16 -- [H][V / 16][D][16], a workgroup's 16
  // columns contiguous -- so that every 128-byte line of the state is read and written by ONE workgroup; in the
  // plain layout two workgroups (often on different L2s) would each pull the whole line for their 64 bytes of it.
  const bool tiled = p.V % kScanCols == 0;
  const int64_t rs = tiled ? kScanCols : p.V;  // floats between two rows of this lane's column
  const int64_t col_off = tiled ? (int64_t)blockIdx.x * D * kScanCols + c : j;
  const int64_t entry = (int64_t)p.H * D * p.V;
  float* to = p.state + p.state_slot[seq] * entry + (int64_t)h * D * p.V + col_off;
  const float* from = p.ctx_len[seq] - ql == 0 ? nullptr : to;  // a sequence's first step starts from zeros
  float S[DPT];
#pragma unroll
  for (int i = 0; i < DPT; ++i) S[i] = (from && col_on && d0 + i < D) ? from[(d0 + i) * rs] : 0.0f;
  const float fixed = p.decay_kind == 1 ? p.decay[h] : 1.0f;
  float nk[E], nq[E], na[E], nv[TB], nsc0 = 0.f, nsc1 = fixed;
  auto request = [&](int b) {  // block b (tokens [b TB, b TB + TB)) into registers
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
    for (int t = 0; t < TB; ++t)
      nv[t] = (col_on && t0 + t < ql) ? p.v[(int64_t)(row0 + t0 + t) * p.ldv + h * p.V + j] : 0.0f;
    if (tid < TB && t0 + tid < ql) {
      const int64_t row = row0 + t0 + tid;
      if (DELTA) nsc0 = p.beta[row * p.ldb + h];
      if (p.decay_kind == 2) nsc1 = p.decay[row * p.ldd + h];
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
  // one token: updates S, leaves this wave's share of the token's read-out in opart
  auto token = [&](int buf, int t, float v) {
    const float* kb = ks + (buf * TB + t) * Dp + d0;
    const float* qb = qs + (buf * TB + t) * Dp + d0;
    if (chan) {
      const float* ab = as + (buf * TB + t) * Dp + d0;
#pragma unroll
      for (int i = 0; i < DPT; ++i) S[i] *= ab[i];
    } else if (p.decay_kind != 0) {
      const float sa = sc[(buf * 2 + 1) * TB + t];
#pragma unroll
      for (int i = 0; i < DPT; ++i) S[i] *= sa;
    }
    float u = v;
    if (DELTA) {
      float part = 0.f;
#pragma unroll
      for (int i = 0; i < DPT; ++i) part += S[i] * kb[i];
      part = rows4_sum(part);  // the wave's RW rows
      if (R > 1) {  // two alternating strips: a strip is rewritten two tokens later, after a barrier in between
        float* ps = part_s + (t & 1) * R * kScanCols;
        if (dg == 0) ps[r * kScanCols + c] = part;
        lds_barrier();
        part = 0.f;
        for (int w = 0; w < R; ++w) part += ps[w * kScanCols + c];
      }
      u = sc[(buf * 2 + 0) * TB + t] * (v - part);
    }
    float o = 0.f;
#pragma unroll
    for (int i = 0; i < DPT; ++i) {
      S[i] += kb[i] * u;
      o += S[i] * qb[i];
    }
    o = rows4_sum(o);
    if (dg == 0) opart[(t * R + r) * kScanCols + c] = o;
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
    lds_barrier();                        // this block's staging is visible; the previous block's opart has been read
    const int nt = ql - b * TB < TB ? ql - b * TB : TB;
    if (nt == TB) {  // a full block: no branches between its tokens
#pragma unroll
      for (int t = 0; t < TB; ++t) token(buf, t, cv[t]);
    } else {
#pragma unroll
      for (int t = 0; t < TB; ++t)
        if (t < nt) token(buf, t, cv[t]);  // uniform
    }
    lds_barrier();  // the block's partial read-outs are complete; its staged inputs have been read
    // the block's [nt][16] outputs, one per thread
    for (int idx = tid; idx < nt * kScanCols; idx += nthreads) {
      const int t = idx / kScanCols, cc = idx % kScanCols;
      float o = 0.f;
      for (int w = 0; w < R; ++w) o += opart[(t * R + w) * kScanCols + cc];
      const int jj = blockIdx.x * kScanCols + cc;
      if (jj < p.V) p.out[((int64_t)(row0 + b * TB + t) * p.H + h) * p.V + jj] = o;
    }
    if (b + 1 < nblocks) stage(buf ^ 1);
  }
#pragma unroll
  for (int i = 0; i < DPT; ++i)
    if (col_on && d0 + i < D) to[(d0 + i) * rs] = S[i];
}

// ---------------------------------------------------------------------------------------------------------------------
// Prompt portions: the same recurrence with every sum over D INSIDE a wave.  A wave owns 4 columns of one (sequence,
// head) and all D rows of them: lane (c, dg) holds rows dg DPT + i of column c (16 lane groups, DPT = D / 16 rounded
// up to a power of two), a dot product over D is DPT FMAs per lane, two row rotations inside each 16-lane row and
// two row swaps -- no LDS, no barrier, also for the delta rule.  The four waves of a workgroup own 16 adjacent columns
// (one tile of the state entry) and share the head's staged k, q and decays; the only workgroup barrier is per token
// block.  With rows spread this thin the chain per token is short enough that the walk is no longer dominated by the
// delta rule's cross-wave sum; the state is touched in 16-byte pieces, which a prompt portion does once.
template <int CTRL>
DEV float dpp_rot(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
// sum over the 16 lane groups of a wave (lanes with the same lane & 3): quads of a 16-lane row, then the four rows
DEV float groups16_sum(float v) {
  v += dpp_rot<0x128>(v);  // row_ror:8
  v += dpp_rot<0x124>(v);  // row_ror:4
  return rows4_sum(v);
}

template <int DPT>
DEV float dot_dpt(const float* S, const float* x) {
  if constexpr (DPT >= 4) {
    float a0 = 0.f, a1 = 0.f;
#pragma unroll
    for (int i = 0; i < DPT; i += 2) {
      a0 += S[i] * x[i];
      a1 += S[i + 1] * x[i + 1];
    }
    return a0 + a1;
  } else {
    float a = 0.f;
#pragma unroll
    for (int i = 0; i < DPT; ++i) a += S[i] * x[i];
    return a;
  }
}

template <int DPT, int TB, bool DELTA>
__global__ __launch_bounds__(256) void matrix_scan_wave_kernel(MatrixScanParams p) {
  constexpr int Dp = 16 * DPT;       // rows of S a wave holds (>= D; rows past D stay zero)
  constexpr int E = TB * Dp / 256;   // staged elements of k (and q, a) per thread and block
  static_assert(E >= 1 && E * 256 == TB * Dp, "a block's staging divides evenly over the workgroup");
  extern __shared__ __align__(16) float lds[];
  const int seq = blockIdx.z, h = blockIdx.y;
  const int ql = p.q_len[seq];
  if (ql <= 0) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c = lane & 3, dg = lane >> 2;
  const int j = blockIdx.x * kScanCols + 4 * wave + c;
  const bool col_on = j < p.V;
  const int g = h / (p.H / p.G);
  const int D = p.D;
  const int d0 = dg * DPT;
  const bool chan = p.decay_kind == 3;
  // LDS: k[2][TB][Dp] | q[2][TB][Dp] | (a[2][TB][Dp]) | sc[2][2][TB] (beta, scalar decay)
  float* ks = lds;
  float* qs = ks + 2 * TB * Dp;
  float* as = qs + 2 * TB * Dp;
  float* sc = as + (chan ? 2 * TB * Dp : 0);
  const int row0 = p.q_start[seq];
  const bool tiled = p.V % kScanCols == 0;  // the state entry's layout: see matrix_scan_kernel
  const int64_t rs = tiled ? kScanCols : p.V;
  const int64_t col_off = tiled ? (int64_t)blockIdx.x * D * kScanCols + 4 * wave + c : j;
  const int64_t entry = (int64_t)p.H * D * p.V;
  const float* from;
  float* to;
  if (p.src_idx) {
    const int si = p.src_idx[seq], di = p.dst_idx[seq];
    from = si >= 0 ? p.src + si * entry + (int64_t)h * D * p.V + col_off : nullptr;
    to = di >= 0 ? p.dst + di * entry + (int64_t)h * D * p.V + col_off : nullptr;
  } else {
    to = p.state + p.state_slot[seq] * entry + (int64_t)h * D * p.V + col_off;
    from = p.ctx_len[seq] - ql == 0 ? nullptr : to;
  }
  float S[DPT], P[DPT];
#pragma unroll
  for (int i = 0; i < DPT; ++i) {
    S[i] = (from && col_on && d0 + i < D) ? from[(d0 + i) * rs] : 0.0f;
    P[i] = 1.0f;
  }
  const float fixed = p.decay_kind == 1 ? p.decay[h] : 1.0f;
  float nk[E], nq[E], na[E], nv[TB], nsc0 = 0.f, nsc1 = fixed;
  auto request = [&](int b) {  // block b (tokens [b TB, b TB + TB)) into registers
    const int t0 = b * TB;
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int idx = e * 256 + tid;
      const int t = idx / Dp, d = idx % Dp;
      const bool on = t0 + t < ql && d < D;  // padded channels and tokens past the end are staged as k = q = 0, a = 1
      const int64_t row = row0 + t0 + t;
      nk[e] = on ? p.k[row * p.ldk + g * D + d] : 0.0f;
      nq[e] = on ? p.q[row * p.ldq + g * D + d] * p.q_scale : 0.0f;
      na[e] = (on && chan) ? p.decay[row * p.ldd + h * D + d] : 1.0f;
    }
#pragma unroll
    for (int t = 0; t < TB; ++t)
      nv[t] = (col_on && t0 + t < ql) ? p.v[(int64_t)(row0 + t0 + t) * p.ldv + h * p.V + j] : 0.0f;
    if (tid < TB && t0 + tid < ql) {
      const int64_t row = row0 + t0 + tid;
      if (DELTA) nsc0 = p.beta[row * p.ldb + h];
      if (p.decay_kind == 2) nsc1 = p.decay[row * p.ldd + h];
    }
  };
  auto stage = [&](int buf) {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int idx = e * 256 + tid;
      ks[buf * TB * Dp + idx] = nk[e];
      qs[buf * TB * Dp + idx] = nq[e];
      if (chan) as[buf * TB * Dp + idx] = na[e];
    }
    if (tid < TB) {
      sc[(buf * 2 + 0) * TB + tid] = nsc0;
      sc[(buf * 2 + 1) * TB + tid] = nsc1;
    }
  };
  auto token = [&](int buf, int t, float v) -> float {  // updates S, returns the column's read-out (in all its lanes)
    const float* kb = ks + (buf * TB + t) * Dp + d0;
    const float* qb = qs + (buf * TB + t) * Dp + d0;
    if (chan) {
      const float* ab = as + (buf * TB + t) * Dp + d0;
#pragma unroll
      for (int i = 0; i < DPT; ++i) S[i] *= ab[i];
      if (p.a_out) {  // uniform: the chunk's decay product for the carry
#pragma unroll
        for (int i = 0; i < DPT; ++i) P[i] *= ab[i];
      }
    } else if (p.decay_kind != 0) {
      const float sa = sc[(buf * 2 + 1) * TB + t];
#pragma unroll
      for (int i = 0; i < DPT; ++i) S[i] *= sa;
    }
    float u = v;
    if (DELTA) u = sc[(buf * 2 + 0) * TB + t] * (v - groups16_sum(dot_dpt<DPT>(S, kb)));
#pragma unroll
    for (int i = 0; i < DPT; ++i) S[i] += kb[i] * u;
    return groups16_sum(dot_dpt<DPT>(S, qb));
  };
  const int nblocks = (ql + TB - 1) / TB;
  request(0);
  stage(0);
  const bool writer = dg == 0 && col_on && !p.no_out;
  for (int b = 0; b < nblocks; ++b) {
    const int buf = b & 1;
    float cv[TB];
#pragma unroll
    for (int t = 0; t < TB; ++t) cv[t] = nv[t];
    if (b + 1 < nblocks) request(b + 1);  // in flight while this block is walked
    lds_barrier();                        // this block's staging is visible; the other buffer has been read
    float* out = p.out + ((int64_t)(row0 + b * TB) * p.H + h) * p.V + j;
    if (ql - b * TB >= TB) {  // a full block: no branches between its tokens
#pragma unroll
      for (int t = 0; t < TB; ++t) {
        const float o = token(buf, t, cv[t]);
        if (writer) out[(int64_t)t * p.H * p.V] = o;
      }
    } else {
      const int nt = ql - b * TB;
#pragma unroll
      for (int t = 0; t < TB; ++t) {
        if (t < nt) {  // uniform
          const float o = token(buf, t, cv[t]);
          if (writer) out[(int64_t)t * p.H * p.V] = o;
        }
      }
    }
    if (b + 1 < nblocks) stage(buf ^ 1);  // that buffer was last read in block b - 1, before this block's barrier
  }
  if (to) {
#pragma unroll
    for (int i = 0; i < DPT; ++i)
      if (col_on && d0 + i < D) to[(d0 + i) * rs] = S[i];
  }
  if (p.a_out && chan && blockIdx.x == 0 && wave == 0 && c == 0) {
#pragma unroll
    for (int i = 0; i < DPT; ++i)
      if (d0 + i < D) p.a_out[((int64_t)seq * p.H + h) * D + d0 + i] = P[i];
  }
}

template <int DPT, int TB>
hipError_t launch_wave(const MatrixScanParams& p, hipStream_t st) {
  constexpr int Dp = 16 * DPT;
  dim3 grid((p.V + kScanCols - 1) / kScanCols, p.H, p.nseq);
  const size_t lds = (size_t)((p.decay_kind == 3 ? 6 : 4) * TB * Dp + 4 * TB) * sizeof(float);
  if (lds > 64 * 1024 || p.D > Dp) return hipErrorInvalidValue;
  if (p.beta) hipLaunchKernelGGL((matrix_scan_wave_kernel<DPT, TB, true>), grid, dim3(256), lds, st, p);
  else hipLaunchKernelGGL((matrix_scan_wave_kernel<DPT, TB, false>), grid, dim3(256), lds, st, p);
  return hipGetLastError();
}

// S_in of every chunk of a sequence: S_in[0] = the slot's state (zeros at position 0), S_in[c + 1] = A_c S_in[c] + B_c
// with B_c the chunk's end state from zeros (found in its scratch entry, which then receives S_in[c]) and A_c the
// product of its decays.  One thread per state element; a sequence has a handful of chunks.
__global__ __launch_bounds__(256) void scan_carry_kernel(ScanCarryParams p) {
  const int seq = blockIdx.z, h = blockIdx.y;
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t DV = (int64_t)p.D * p.V;
  const int n = p.s_count[seq];
  if (e >= DV || n <= 0 || p.q_len[seq] <= 0) return;
  const int d = p.V % kScanCols == 0 ? (int)((e / kScanCols) % p.D) : (int)(e / p.V);  // tile-major or plain entries
  const bool fresh = p.ctx_len[seq] - p.q_len[seq] == 0;
  float S = fresh ? 0.0f : p.state[((int64_t)p.state_slot[seq] * p.H + h) * DV + e];
  const float fixed = p.decay_kind == 1 ? p.decay[h] : 1.0f;
  const int c0 = p.s_first[seq];
  for (int i = 0; i < n; ++i) {
    const int cid = c0 + i;
    float* slot = p.scratch + ((int64_t)cid * p.H + h) * DV + e;
    const float B = *slot;
    *slot = S;
    if (i + 1 < n) {
      float a = 1.0f;
      if (p.decay_kind == 3) a = p.a_chunk[((int64_t)cid * p.H + h) * p.D + d];
      else if (p.decay_kind == 1)
        for (int t = 0; t < p.cq_len[cid]; ++t) a *= fixed;  // the product the walk itself would form
      S = a * S + B;
    }
  }
}

template <int DPT, int TB>
hipError_t launch(const MatrixScanParams& p, hipStream_t st) {
  constexpr int RW = 4 * DPT;
  const int R = (p.D + RW - 1) / RW;
  const int Dp = R * RW;
  dim3 grid((p.V + kScanCols - 1) / kScanCols, p.H, p.nseq);
  const size_t lds = (size_t)((p.decay_kind == 3 ? 6 : 4) * TB * Dp + 4 * TB + 2 * R * kScanCols + TB * R * kScanCols) *
                     sizeof(float);
  if (lds > 64 * 1024 || R > 16) return hipErrorInvalidValue;
  if (p.beta) hipLaunchKernelGGL((matrix_scan_kernel<DPT, TB, true>), grid, dim3(R * 64), lds, st, p, R);
  else hipLaunchKernelGGL((matrix_scan_kernel<DPT, TB, false>), grid, dim3(R * 64), lds, st, p, R);
  return hipGetLastError();
}

}  // namespace
}  // namespace dsse

extern "C" hipError_t dsse_matrix_scan(const dsse::MatrixScanParams* p, hipStream_t st) {
  if (p->nseq <= 0 || p->H <= 0) return hipSuccess;
  if (p->D < 1 || p->D > 512 || p->V < 1 || p->G < 1 || p->H % p->G) return hipErrorInvalidValue;
  if (p->portions || p->src_idx) {  // prompt portions (and every pass of the two-level walk): all sums inside a wave (rows per lane = D / 16 rounded up to a power of two)
    if (p->D <= 16) return dsse::launch_wave<1, 16>(*p, st);
    if (p->D <= 32) return dsse::launch_wave<2, 16>(*p, st);
    if (p->D <= 64) return dsse::launch_wave<4, 16>(*p, st);
    if (p->D <= 128) return dsse::launch_wave<8, 16>(*p, st);
    if (p->D <= 256) return dsse::launch_wave<16, 8>(*p, st);
    return dsse::launch_wave<32, 4>(*p, st);
  }
  // rows of S per lane (a wave holds 4 DPT rows of 16 columns, a workgroup up to 16 waves) and tokens per block (as
  // long as 64 KB of LDS allow)
  if (p->D <= 64) return dsse::launch<2, 16>(*p, st);
  if (p->D <= 128) return dsse::launch<4, 16>(*p, st);
  if (p->D <= 256) return dsse::launch<4, 8>(*p, st);
  return dsse::launch<8, 4>(*p, st);
}

extern "C" hipError_t dsse_scan_carry(const dsse::ScanCarryParams* p, hipStream_t st) {
  if (p->nseq <= 0 || p->H <= 0) return hipSuccess;
  const long long dv = (long long)p->D * p->V;
  hipLaunchKernelGGL(dsse::scan_carry_kernel, dim3((unsigned)((dv + 255) / 256), p->H, p->nseq), dim3(256), 0, st, *p);
  return hipGetLastError();
}
