// Latent (compressed-KV) attention with a sliding window over the engine's paged cache.
//
// The cache holds, per token and layer, one row [normed latent c (rk) | rotated shared key part (dr)] -- nothing per
// head.  Attention runs in the folded form: with q_abs[h] = W_uk[h]^T q_unrotated[h] (a per-head GEMM before this
// kernel), the score of head h against token j is (q_abs[h] . c_j + rot(q_rot[h]) . kr_j) * scale, and the head's output
// is W_uv[h] (sum_j p_j c_j) (a per-head GEMM after it).  So every head reads the same rk + dr numbers per key and the
// kernel is multi-query attention with key width rk + dr and value width rk.
//
//   latent_kv_write   c = rms-norm(down-projection[:rk]) * w, kr = rot(down-projection[rk:]) -> cache row of the token
//   latent_attention  generic row kernel (any element type, any sizes): one workgroup per (query tile, head), the
//                     tile's rows one after the other; keys max(0, pos - window + 1) .. pos through the block table,
//                     256 keys per pass (one key per thread for the scores, one latent coordinate per thread for the
//                     weighted sum), online softmax in fp32.  Decode is a one-row tile.
//
// Rotation: interleaved pairs (2i, 2i + 1) of the rotated part, angle from a host-made fp32 (cos, sin) table per
// position that already carries the frequency scaling and amplitude of the design.
#include "api_layers.h"

namespace dsse {
namespace {

DEV float block_reduce_sum(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float s = 0.f;
  for (int i = 0; i < (int)(blockDim.x >> 6); ++i) s += red[i];
  return s;
}
DEV float block_reduce_max(float v, float* red) {
  v = wave_max(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float s = red[0];
  for (int i = 1; i < (int)(blockDim.x >> 6); ++i) s = fmaxf(s, red[i]);
  return s;
}

template <typename T>
__global__ __launch_bounds__(256) void latent_kv_write_kernel(LatentKvWriteParams p) {
  __shared__ float red[4];
  const int row = blockIdx.x;
  const int slot = p.slots[row];
  if (slot < 0 || slot >= p.num_slots) return;  // uniform per workgroup
  const int D = p.rk + p.dr;
  const float* src = p.ckr + (int64_t)row * D;
  T* dst = reinterpret_cast<T*>(p.cache) + (int64_t)slot * D;
  float ss = 0.f;
  for (int d = threadIdx.x; d < p.rk; d += blockDim.x) ss += src[d] * src[d];
  ss = block_reduce_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)p.rk + p.eps);
  const T* nw = reinterpret_cast<const T*>(p.norm_w);
  for (int d = threadIdx.x; d < p.rk; d += blockDim.x) dst[d] = (T)(src[d] * inv * (float)nw[d]);
  int pos = p.positions[row];
  pos = pos < 0 ? 0 : (pos >= p.rope_len ? p.rope_len - 1 : pos);
  const float2* cs = p.rope + (int64_t)pos * (p.dr / 2);
  for (int i = threadIdx.x; i < p.dr / 2; i += blockDim.x) {
    const float u = src[p.rk + 2 * i], v = src[p.rk + 2 * i + 1];
    const float2 a = cs[i];
    dst[p.rk + 2 * i] = (T)(u * a.x - v * a.y);
    dst[p.rk + 2 * i + 1] = (T)(v * a.x + u * a.y);
  }
}

constexpr int kAccMax = 4;  // latent coordinates per thread: rk <= 1024

template <typename T>
__global__ __launch_bounds__(256) void latent_attention_rows_kernel(LatentAttnParams p) {
  extern __shared__ float smem[];
  const int D = p.rk + p.dr;
  float* qv = smem;               // [D]
  float* sc = smem + D;           // [256] scores, then weights
  int* sl = reinterpret_cast<int*>(sc + 256);  // [256] cache rows of the pass's keys
  float* red = reinterpret_cast<float*>(sl + 256);  // [4]
  const int tid = threadIdx.x;
  const int seq = p.work_seq[blockIdx.x], tile = p.work_tile[blockIdx.x], h = blockIdx.y;
  const int ql = p.q_len[seq];
  const int* bt = p.block_tables + (int64_t)seq * p.max_blocks;
  const T* cache = reinterpret_cast<const T*>(p.cache);
  for (int i = 0; i < p.qt; ++i) {
    const int off = tile * p.qt + i;
    if (off >= ql) break;  // uniform
    const int row = p.q_start[seq] + off;
    const int pos = p.ctx_len[seq] - ql + off;
    __syncthreads();
    for (int d = tid; d < p.rk; d += 256) qv[d] = p.q_abs[((int64_t)row * p.H + h) * p.rk + d];
    {
      const T* qr = reinterpret_cast<const T*>(p.q) + ((int64_t)row * p.H + h) * (p.dn + p.dr) + p.dn;
      const int pp = pos < 0 ? 0 : (pos >= p.rope_len ? p.rope_len - 1 : pos);
      const float2* cs = p.rope + (int64_t)pp * (p.dr / 2);
      for (int k = tid; k < p.dr / 2; k += 256) {
        const float u = (float)qr[2 * k], v = (float)qr[2 * k + 1];
        const float2 a = cs[k];
        qv[p.rk + 2 * k] = u * a.x - v * a.y;
        qv[p.rk + 2 * k + 1] = v * a.x + u * a.y;
      }
    }
    __syncthreads();
    const int lo = pos - p.window + 1 > 0 ? pos - p.window + 1 : 0;
    float m = -INFINITY, l = 0.f;
    float acc[kAccMax];
#pragma unroll
    for (int a = 0; a < kAccMax; ++a) acc[a] = 0.f;
    for (int kb = lo; kb <= pos; kb += 256) {
      const int j = kb + tid;
      float s = -INFINITY;
      int slot = 0;
      if (j <= pos) {
        int blk = bt[j / kBS];
        blk = (unsigned)blk < (unsigned)p.num_blocks ? blk : 0;  // a stale table entry never leaves the cache
        slot = blk * kBS + j % kBS;
        const T* e = cache + (int64_t)slot * D;
        float dot = 0.f;
        for (int d = 0; d < D; ++d) dot += qv[d] * (float)e[d];
        s = dot * p.scale;
      }
      sl[tid] = slot;
      const float bm = block_reduce_max(s, red);
      const float mn = fmaxf(m, bm);
      const float corr = m == -INFINITY ? 0.f : expf(m - mn);
      const float pj = j <= pos ? expf(s - mn) : 0.f;
      sc[tid] = pj;
      const float bs = block_reduce_sum(pj, red);  // its barriers also publish sc / sl
      l = l * corr + bs;
      m = mn;
      const int nk = pos - kb + 1 < 256 ? pos - kb + 1 : 256;
#pragma unroll
      for (int a = 0; a < kAccMax; ++a) {
        const int d = tid + 256 * a;
        if (d < p.rk) {
          float v = acc[a] * corr;
          for (int jj = 0; jj < nk; ++jj) v += sc[jj] * (float)cache[(int64_t)sl[jj] * D + d];
          acc[a] = v;
        }
      }
      __syncthreads();
    }
    T* out = reinterpret_cast<T*>(p.out) + ((int64_t)row * p.H + h) * p.rk;
    const float inv = 1.0f / l;
#pragma unroll
    for (int a = 0; a < kAccMax; ++a) {
      const int d = tid + 256 * a;
      if (d < p.rk) out[d] = (T)(acc[a] * inv);
    }
  }
}

}  // namespace
}  // namespace dsse

extern "C" hipError_t dsse_latent_kv_write(const dsse::LatentKvWriteParams* p, hipStream_t st) {
  if (p->T <= 0) return hipSuccess;
  if (p->f32) hipLaunchKernelGGL(dsse::latent_kv_write_kernel<float>, dim3(p->T), dim3(256), 0, st, *p);
  else hipLaunchKernelGGL(dsse::latent_kv_write_kernel<bf16>, dim3(p->T), dim3(256), 0, st, *p);
  return hipGetLastError();
}

extern "C" hipError_t dsse_latent_attention(int num_work, const dsse::LatentAttnParams* p, hipStream_t st) {
  if (num_work <= 0) return hipSuccess;
  if (p->rk > 256 * dsse::kAccMax) return hipErrorInvalidValue;
  const size_t lds = sizeof(float) * (p->rk + p->dr + 256 + 256 + 4);
  dim3 grid(num_work, p->H);
  if (p->f32) hipLaunchKernelGGL(dsse::latent_attention_rows_kernel<float>, grid, dim3(256), lds, st, *p);
  else hipLaunchKernelGGL(dsse::latent_attention_rows_kernel<bf16>, grid, dim3(256), lds, st, *p);
  return hipGetLastError();
}
