// One-number RMS norm on a sublayer's OUTPUT ("sandwich" residual: stream += y / rms(y) * g) and the embedding gather
// into an fp32 residual stream.  The stream is fp32; the kernels also emit its rounding to the element type, which is
// what the next projection reads (the sublayers of such designs read the stream itself, with no norm before them).
// One workgroup per row; mean(y^2) and the scaling in fp32.
#include "api_layers.h"

namespace dsse {
namespace {

DEV float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[wave] = v;
  __syncthreads();
  float s = 0.f;
  for (int i = 0; i < nw; ++i) s += red[i];
  return s;
}

template <typename T>
__global__ __launch_bounds__(256) void scalar_norm_kernel(ScalarNormParams p) {
  __shared__ float red[4];
  const int row = blockIdx.x;
  float* resid = p.resid + (int64_t)row * p.W;
  const int ns = p.mode == 0 ? p.nsum : 1;
  const float* src = p.mode == 0 ? p.y + (int64_t)row * ns * p.W : resid;
  T* xb = reinterpret_cast<T*>(p.xb) + (int64_t)row * p.W;
  float ss = 0.f;
  for (int d = threadIdx.x; d < p.W; d += blockDim.x) {
    float v = src[d];
    for (int s = 1; s < ns; ++s) v += src[(int64_t)s * p.W + d];  // the same order in both passes
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float s = (float)reinterpret_cast<const T*>(p.g)[0] / sqrtf(ss / (float)p.W + p.eps);
  for (int d = threadIdx.x; d < p.W; d += blockDim.x) {
    if (p.mode == 0) {
      float y = src[d];
      for (int k = 1; k < ns; ++k) y += src[(int64_t)k * p.W + d];
      const float v = resid[d] + y * s;
      resid[d] = v;
      xb[d] = (T)v;
    } else {
      xb[d] = (T)(src[d] * s);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void embed_rows_kernel(int W, int vocab, const int* ids, const T* embed, float* resid,
                                                         T* xb) {
  const int row = blockIdx.x;
  int id = ids[row];
  id = (unsigned)id < (unsigned)vocab ? id : 0;  // padded / inactive rows carry any id
  const T* e = embed + (int64_t)id * W;
  for (int d = threadIdx.x; d < W; d += blockDim.x) {
    const T v = e[d];
    resid[(int64_t)row * W + d] = (float)v;
    xb[(int64_t)row * W + d] = v;
  }
}

}  // namespace
}  // namespace dsse

extern "C" hipError_t dsse_scalar_norm(const dsse::ScalarNormParams* p, hipStream_t st) {
  if (p->M <= 0) return hipSuccess;
  if (p->f32) hipLaunchKernelGGL(dsse::scalar_norm_kernel<float>, dim3(p->M), dim3(256), 0, st, *p);
  else hipLaunchKernelGGL(dsse::scalar_norm_kernel<bf16>, dim3(p->M), dim3(256), 0, st, *p);
  return hipGetLastError();
}

extern "C" hipError_t dsse_embed_rows(int M, int W, int vocab, const int* ids, const void* embed, float* resid, void* xb,
                                      int f32, hipStream_t st) {
  if (M <= 0) return hipSuccess;
  if (f32)
    hipLaunchKernelGGL(dsse::embed_rows_kernel<float>, dim3(M), dim3(256), 0, st, W, vocab, ids,
                       reinterpret_cast<const float*>(embed), resid, reinterpret_cast<float*>(xb));
  else
    hipLaunchKernelGGL(dsse::embed_rows_kernel<bf16>, dim3(M), dim3(256), 0, st, W, vocab, ids,
                       reinterpret_cast<const bf16*>(embed), resid, reinterpret_cast<bf16*>(xb));
  return hipGetLastError();
}
