// Several residual streams around a sublayer, layer norm with bias, and two
// small elementwise ops (squared ReLU, tanh soft cap).
//
// A token carries S copies of the residual, x[t, s, :] (fp32). A sublayer
// reads one mixture of them and writes back into all of them:
//
//   u      = sum_s w_in[s] * x[t, s]
//   h      = (u - mean(u)) / sqrt(var(u) + eps) * g + b        (to the GEMM)
//   x[t,j] = sum_s mix[s, j] * x[t, s] + w_out[j] * (a1 * y1 + a2 * y2)
//
// With S = 1, w_in = mix = w_out = 1 this is the plain pre-norm residual.
// One workgroup per token for the read; the write alone is elementwise; the
// model's steady state is the fused kernel (a write and the next read in one
// pass over the token's streams).
#include "hybrid_common.h"

namespace xllm {
namespace hyb {

constexpr int MAX_STREAMS = 8;

template <typename TO>
__global__ void __launch_bounds__(256) streams_mix_norm_kernel(
    TO* __restrict__ out, const float* __restrict__ x,
    const float* __restrict__ w_in, const float* __restrict__ g,
    const float* __restrict__ b, float eps, int S, int W) {
  extern __shared__ float u[];             // [W]
  __shared__ float tmp[16];
  const long t = blockIdx.x;
  const float* xr = x + t * (long)S * W;
  float win[MAX_STREAMS];
#pragma unroll
  for (int s = 0; s < MAX_STREAMS; ++s) win[s] = (w_in && s < S) ? w_in[s] : 1.f;
  float sum = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float a = 0.f;
#pragma unroll
    for (int s = 0; s < MAX_STREAMS; ++s)
      if (s < S) a += win[s] * xr[(long)s * W + c];
    u[c] = a;
    sum += a;
  }
  const float mean = block_reduce_sum(sum, tmp) / (float)W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float d = u[c] - mean;
    ss += d * d;
  }
  __syncthreads();                         // tmp[0] read by all before reuse
  const float var = block_reduce_sum(ss, tmp) / (float)W;
  const float rs = 1.0f / sqrtf(var + eps);
  for (int c = threadIdx.x; c < W; c += blockDim.x)
    IO<TO>::st(out + t * (long)W + c, (u[c] - mean) * rs * g[c] + b[c]);
}

template <typename T>
__global__ void streams_update_kernel(
    float* __restrict__ x, const float* __restrict__ mix,
    const float* __restrict__ w_out, const T* __restrict__ y1, float a1,
    const T* __restrict__ y2, float a2, long tokens, int S, int W) {
  __shared__ float m[MAX_STREAMS * MAX_STREAMS + MAX_STREAMS];
  if (threadIdx.x < S * S) m[threadIdx.x] = mix ? mix[threadIdx.x]
      : ((threadIdx.x / S == threadIdx.x % S) ? 1.f : 0.f);
  if (threadIdx.x < S)
    m[MAX_STREAMS * MAX_STREAMS + threadIdx.x] = w_out ? w_out[threadIdx.x] : 1.f;
  __syncthreads();
  const long n = tokens * (long)W;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < n;
       idx += (long)gridDim.x * blockDim.x) {
    const long t = idx / W;
    const int c = (int)(idx - t * W);
    float* xr = x + t * (long)S * W + c;
    float y = a1 * IO<T>::ld(y1 + idx);
    if (y2) y += a2 * IO<T>::ld(y2 + idx);
    float old[MAX_STREAMS];
#pragma unroll
    for (int s = 0; s < MAX_STREAMS; ++s)
      if (s < S) old[s] = xr[(long)s * W];
#pragma unroll
    for (int j = 0; j < MAX_STREAMS; ++j) {
      if (j < S) {
        float acc = m[MAX_STREAMS * MAX_STREAMS + j] * y;
#pragma unroll
        for (int s = 0; s < MAX_STREAMS; ++s)
          if (s < S) acc += m[s * S + j] * old[s];
        xr[(long)j * W] = acc;
      }
    }
  }
}

// four neighbouring values at once (16 B of fp32, 8 B of bf16)
template <typename T> struct Quad;
template <> struct Quad<float> {
  static XLLM_DEV void ld(const float* p, float v[4]) {
    const float4 x = *reinterpret_cast<const float4*>(p);
    v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
  }
  static XLLM_DEV void st(float* p, const float v[4]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  }
};
template <> struct Quad<unsigned short> {
  static XLLM_DEV void ld(const unsigned short* p, float v[4]) {
    const ushort4_t x = *reinterpret_cast<const ushort4_t*>(p);
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = bf16_to_f32(x.x[i]);
  }
  static XLLM_DEV void st(unsigned short* p, const float v[4]) {
    ushort4_t x;
#pragma unroll
    for (int i = 0; i < 4; ++i) x.x[i] = f32_to_bf16(v[i]);
    *reinterpret_cast<ushort4_t*>(p) = x;
  }
};

// The write of one sublayer fused with the read of the next: a token's streams
// are updated in place and the next sublayer's normed input is produced from
// the new values in the same pass (one workgroup per token). V = 4: four
// columns per thread and access (width a multiple of 4), V = 1: any width.
template <typename T, int V>
__global__ void __launch_bounds__(256) streams_update_mix_norm_kernel(
    T* __restrict__ out, float* __restrict__ x, const float* __restrict__ mix,
    const float* __restrict__ w_out, const T* __restrict__ y1, float a1,
    const T* __restrict__ y2, float a2, const float* __restrict__ w_in,
    const float* __restrict__ g, const float* __restrict__ b, float eps, int S,
    int W) {
  extern __shared__ float u[];             // [W]
  __shared__ float tmp[16];
  __shared__ float m[MAX_STREAMS * MAX_STREAMS + 2 * MAX_STREAMS];
  const int tid = threadIdx.x;
  if (tid < S * S) m[tid] = mix ? mix[tid] : ((tid / S == tid % S) ? 1.f : 0.f);
  if (tid < S) {
    m[MAX_STREAMS * MAX_STREAMS + tid] = w_out ? w_out[tid] : 1.f;
    m[MAX_STREAMS * MAX_STREAMS + MAX_STREAMS + tid] = w_in ? w_in[tid] : 1.f;
  }
  __syncthreads();
  const long t = blockIdx.x;
  float* xr = x + t * (long)S * W;
  float sum = 0.f;
  for (int c = tid * V; c < W; c += blockDim.x * V) {
    float y[V], yb[V], old[MAX_STREAMS][V], a[V];
    if (V == 4) {
      Quad<T>::ld(y1 + t * (long)W + c, y);
      if (y2) Quad<T>::ld(y2 + t * (long)W + c, yb);
    } else {
      y[0] = IO<T>::ld(y1 + t * (long)W + c);
      if (y2) yb[0] = IO<T>::ld(y2 + t * (long)W + c);
    }
#pragma unroll
    for (int i = 0; i < V; ++i) {
      y[i] = a1 * y[i] + (y2 ? a2 * yb[i] : 0.f);
      a[i] = 0.f;
    }
#pragma unroll
    for (int s = 0; s < MAX_STREAMS; ++s) {
      if (s < S) {
        if (V == 4) Quad<float>::ld(xr + (long)s * W + c, old[s]);
        else old[s][0] = xr[(long)s * W + c];
      }
    }
#pragma unroll
    for (int j = 0; j < MAX_STREAMS; ++j) {
      if (j < S) {
        float acc[V];
#pragma unroll
        for (int i = 0; i < V; ++i)
          acc[i] = m[MAX_STREAMS * MAX_STREAMS + j] * y[i];
#pragma unroll
        for (int s = 0; s < MAX_STREAMS; ++s)
          if (s < S) {
#pragma unroll
            for (int i = 0; i < V; ++i) acc[i] += m[s * S + j] * old[s][i];
          }
        if (V == 4) Quad<float>::st(xr + (long)j * W + c, acc);
        else xr[(long)j * W + c] = acc[0];
#pragma unroll
        for (int i = 0; i < V; ++i)
          a[i] += m[MAX_STREAMS * MAX_STREAMS + MAX_STREAMS + j] * acc[i];
      }
    }
#pragma unroll
    for (int i = 0; i < V; ++i) { u[c + i] = a[i]; sum += a[i]; }
  }
  const float mean = block_reduce_sum(sum, tmp) / (float)W;
  float ss = 0.f;
  for (int c = tid * V; c < W; c += blockDim.x * V) {
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const float d = u[c + i] - mean;
      ss += d * d;
    }
  }
  __syncthreads();
  const float var = block_reduce_sum(ss, tmp) / (float)W;
  const float rs = 1.0f / sqrtf(var + eps);
  for (int c = tid * V; c < W; c += blockDim.x * V) {
    float h[V];
#pragma unroll
    for (int i = 0; i < V; ++i)
      h[i] = (u[c + i] - mean) * rs * g[c + i] + b[c + i];
    if (V == 4) Quad<T>::st(out + t * (long)W + c, h);
    else IO<T>::st(out + t * (long)W + c, h[0]);
  }
}

// x <- max(x, 0)^2 in place
template <typename T>
__global__ void relu_sq_kernel(T* __restrict__ x, long n) {
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < n;
       idx += (long)gridDim.x * blockDim.x) {
    const float v = fmaxf(IO<T>::ld(x + idx), 0.f);
    IO<T>::st(x + idx, v * v);
  }
}

// out (fp32) = cap * tanh(x / cap)
template <typename T>
__global__ void softcap_kernel(float* __restrict__ out,
                               const T* __restrict__ x, float cap, long n) {
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < n;
       idx += (long)gridDim.x * blockDim.x)
    out[idx] = cap * tanhf(IO<T>::ld(x + idx) / cap);
}

static inline int blocks_for(long n) {
  const long b = (n + 255) / 256;
  return (int)(b < 65535 ? b : 65535);
}

template <typename TO>
void launch_streams_mix_norm(TO* out, const float* x, const float* w_in,
                             const float* g, const float* b, float eps,
                             int tokens, int S, int W, hipStream_t st) {
  if (tokens == 0) return;
  hipLaunchKernelGGL((streams_mix_norm_kernel<TO>), dim3(tokens), dim3(256),
                     (size_t)W * sizeof(float), st, out, x, w_in, g, b, eps, S,
                     W);
}
template <typename T>
void launch_streams_update(float* x, const float* mix, const float* w_out,
                           const T* y1, float a1, const T* y2, float a2,
                           long tokens, int S, int W, hipStream_t st) {
  if (tokens == 0) return;
  hipLaunchKernelGGL((streams_update_kernel<T>), dim3(blocks_for(tokens * W)),
                     dim3(256), 0, st, x, mix, w_out, y1, a1, y2, a2, tokens,
                     S, W);
}
template <typename T>
void launch_streams_update_mix_norm(T* out, float* x, const float* mix,
                                    const float* w_out, const T* y1, float a1,
                                    const T* y2, float a2, const float* w_in,
                                    const float* g, const float* b, float eps,
                                    int tokens, int S, int W, hipStream_t st) {
  if (tokens == 0) return;
  if (W % 4 == 0)
    hipLaunchKernelGGL((streams_update_mix_norm_kernel<T, 4>), dim3(tokens),
                       dim3(256), (size_t)W * sizeof(float), st, out, x, mix,
                       w_out, y1, a1, y2, a2, w_in, g, b, eps, S, W);
  else
    hipLaunchKernelGGL((streams_update_mix_norm_kernel<T, 1>), dim3(tokens),
                       dim3(256), (size_t)W * sizeof(float), st, out, x, mix,
                       w_out, y1, a1, y2, a2, w_in, g, b, eps, S, W);
}
template <typename T>
void launch_relu_sq(T* x, long n, hipStream_t st) {
  if (n == 0) return;
  hipLaunchKernelGGL((relu_sq_kernel<T>), dim3(blocks_for(n)), dim3(256), 0,
                     st, x, n);
}
template <typename T>
void launch_softcap(float* out, const T* x, float cap, long n,
                    hipStream_t st) {
  if (n == 0) return;
  hipLaunchKernelGGL((softcap_kernel<T>), dim3(blocks_for(n)), dim3(256), 0,
                     st, out, x, cap, n);
}

#define INST_STREAMS(T)                                                       \
  template void launch_streams_mix_norm<T>(T*, const float*, const float*,    \
                                           const float*, const float*, float, \
                                           int, int, int, hipStream_t);       \
  template void launch_streams_update<T>(float*, const float*, const float*,  \
                                         const T*, float, const T*, float,    \
                                         long, int, int, hipStream_t);        \
  template void launch_streams_update_mix_norm<T>(                            \
      T*, float*, const float*, const float*, const T*, float, const T*,      \
      float, const float*, const float*, const float*, float, int, int, int,  \
      hipStream_t);                                                           \
  template void launch_relu_sq<T>(T*, long, hipStream_t);                     \
  template void launch_softcap<T>(float*, const T*, float, long, hipStream_t);
INST_STREAMS(float)
INST_STREAMS(unsigned short)

}  // namespace hyb
}  // namespace xllm
