// Routed-expert support kernels: the router's selection (sigmoid scores,
// group-limited top-k over fp32 logits) and the weighted combine of expert outputs. The
// expert matrix products themselves are library GEMMs.
#include "hybrid_common.h"

namespace xllm {
namespace hyb {

// One wavefront per token; z [T, E] are the fp32 router logits (an fp32 GEMM
// upstream), scores = sigmoid(z).
// Experts form n_groups equal neighbouring groups; a group's score is the
// sum of its two largest scores; only the `keep` best groups are eligible.
// ids/weights [T, top]: the eligible experts with the largest scores, weights
// are the raw scores. Ties go to the lower index.
__global__ void moe_route_kernel(int* __restrict__ ids,
                                 float* __restrict__ wts,
                                 const float* __restrict__ z, int E, int top,
                                 int n_groups, int keep) {
  extern __shared__ float smem[];
  float* sc = smem;                 // [E] scores
  float* el = sc + E;               // [E] eligible score or -1 (taken/masked)
  float* gsc = el + E;              // [n_groups]
  const int t = blockIdx.x;
  const int lane = threadIdx.x;
  for (int e = lane; e < E; e += 64) sc[e] = sigmoidf_(z[(long)t * E + e]);
  __syncthreads();
  const int gsz = E / n_groups;
  if (n_groups > 1) {
    for (int g = lane; g < n_groups; g += 64) {
      float a = -1.f, b = -1.f;      // two largest (scores are in (0,1))
      for (int i = 0; i < gsz; ++i) {
        const float x = sc[g * gsz + i];
        if (x > a) { b = a; a = x; } else if (x > b) { b = x; }
      }
      gsc[g] = a + (gsz > 1 ? b : 0.f);
    }
    __syncthreads();
    for (int e = lane; e < E; e += 64) el[e] = -1.f;
    __syncthreads();
    if (lane == 0) {
      for (int kk = 0; kk < keep; ++kk) {
        int best = -1; float bv = -INFINITY;
        for (int g = 0; g < n_groups; ++g)
          if (gsc[g] > bv) { bv = gsc[g]; best = g; }
        if (best < 0) break;
        gsc[best] = -INFINITY;
        for (int i = 0; i < gsz; ++i) el[best * gsz + i] = sc[best * gsz + i];
      }
    }
    __syncthreads();
  } else {
    for (int e = lane; e < E; e += 64) el[e] = sc[e];
    __syncthreads();
  }
  for (int kk = 0; kk < top; ++kk) {
    float bv = -1.f; int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64)
      if (el[e] > bv) { bv = el[e]; bi = e; }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ov = __shfl_xor(bv, off, 64);
      const int oi = __shfl_xor(bi, off, 64);
      if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    if (bi == 0x7fffffff) bi = 0;   // fewer eligible experts than top
    if (lane == 0) {
      ids[(long)t * top + kk] = bi;
      wts[(long)t * top + kk] = sc[bi];
      el[bi] = -1.f;
    }
    __syncthreads();
  }
}

// out[t, c] = sum_k wts[t, k] * y[rows[t, k], c]      (fp32 accumulate)
template <typename T>
__global__ void moe_combine_kernel(float* __restrict__ out,
                                   const T* __restrict__ y,
                                   const int* __restrict__ rows,
                                   const float* __restrict__ wts, long tokens,
                                   int width, int top) {
  const long n = tokens * (long)width;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < n;
       idx += (long)gridDim.x * blockDim.x) {
    const long t = idx / width;
    const int c = (int)(idx - t * width);
    float a = 0.f;
    for (int kk = 0; kk < top; ++kk)
      a += wts[t * top + kk] *
           IO<T>::ld(y + (long)rows[t * top + kk] * width + c);
    out[idx] = a;
  }
}

void launch_moe_route(int* ids, float* wts, const float* z, int tokens, int E,
                      int top, int n_groups, int keep, hipStream_t st) {
  if (tokens == 0) return;
  const size_t lds = (size_t)(2 * E + n_groups) * sizeof(float);
  hipLaunchKernelGGL(moe_route_kernel, dim3(tokens), dim3(64), lds, st, ids,
                     wts, z, E, top, n_groups, keep);
}

template <typename T>
void launch_moe_combine(float* out, const T* y, const int* rows,
                        const float* wts, long tokens, int width, int top,
                        hipStream_t st) {
  const long n = tokens * (long)width;
  if (n == 0) return;
  const int blocks = (int)((n + 255) / 256 < 65535 ? (n + 255) / 256 : 65535);
  hipLaunchKernelGGL((moe_combine_kernel<T>), dim3(blocks), dim3(256), 0, st,
                     out, y, rows, wts, tokens, width, top);
}

#define INST_MOE(T)                                                          \
  template void launch_moe_combine<T>(float*, const T*, const int*,          \
                                      const float*, long, int, int,          \
                                      hipStream_t);
INST_MOE(float)
INST_MOE(unsigned short)

}  // namespace hyb
}  // namespace xllm
