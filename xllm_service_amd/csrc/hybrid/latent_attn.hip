// Latent attention over a paged cache of shared rows [latent c | rotated key].
//
// Every head's key is a linear image of the same cached latent, so queries
// arrive already folded through the key up-projection: a query row is
// [q_abs (kv_rank) | q_rot (rot)] and scores are plain dot products with the
// cached row. Values are the latent itself (first kv_rank entries of the
// row); the value up-projection is applied by the caller afterwards.
//
// Scores, softmax weights and the weighted sum are fp32. One wavefront per
// (query token, head): 64 keys are scored per step, one per lane, then the
// lanes switch to owning output columns for the weighted sum.
#include "hybrid_common.h"

namespace xllm {
namespace hyb {

// cache row write: c = rmsnorm(dkv[:r]) * w ; kr = rope(dkv[r:]).
// One wavefront per token.
template <typename T>
__global__ void latent_kv_store_kernel(
    T* __restrict__ cache, const T* __restrict__ dkv,
    const float* __restrict__ norm_w, float eps,
    const long* __restrict__ pos, const double* __restrict__ inv_freq,
    float mscale, int rot_dims, const long* __restrict__ slots, int r, int rd,
    long dkv_stride) {
  const int t = blockIdx.x;
  const long slot = slots[t];
  if (slot < 0) return;
  const int lane = threadIdx.x;
  const T* src = dkv + (long)t * dkv_stride;
  T* dst = cache + slot * (long)(r + rd);
  float ss = 0.f;
  for (int i = lane; i < r; i += 64) {
    float v = IO<T>::ld(src + i);
    ss += v * v;
  }
  ss = wave_reduce_sum(ss);
  const float rs = 1.0f / sqrtf(ss / (float)r + eps);
  for (int i = lane; i < r; i += 64)
    IO<T>::st(dst + i, IO<T>::ld(src + i) * rs * norm_w[i]);
  const int half = rot_dims >> 1;
  for (int i = lane; i < half; i += 64) {
    double s, c;
    sincos((double)pos[t] * inv_freq[i], &s, &c);
    const float cf = (float)c * mscale, sf = (float)s * mscale;
    const float u = IO<T>::ld(src + r + 2 * i);
    const float v = IO<T>::ld(src + r + 2 * i + 1);
    IO<T>::st(dst + r + 2 * i, u * cf - v * sf);
    IO<T>::st(dst + r + 2 * i + 1, v * cf + u * sf);
  }
  for (int i = rot_dims + lane; i < rd; i += 64)
    IO<T>::st(dst + r + i, IO<T>::ld(src + r + i));
}

constexpr int LAT_MAX_ACC = 16;  // kv_rank <= 64 * 16

// q [T, H, W] (W = r + rd), out fp32 [T, H, r].
// cu_q == nullptr: decode (token t is sequence t, sees seq_lens[t] keys);
// else prefill: token t belongs to the sequence s with cu_q[s] <= t <
// cu_q[s+1] and sees seq_lens[s] - (cu_q[s+1] - 1 - t) keys.
template <typename T>
__global__ void latent_attn_kernel(
    float* __restrict__ out, const T* __restrict__ q,
    const T* __restrict__ cache, const int* __restrict__ block_tables,
    const int* __restrict__ cu_q, const int* __restrict__ seq_lens,
    int n_seqs, int heads, int r, int rd, int block_size, int table_width,
    float scale, long q_row_stride) {
  extern __shared__ float smem[];
  const int W = r + rd;
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  const int h = blockIdx.y * nw + wid;

  int s, n_keys;
  if (cu_q == nullptr) {
    s = t;
    n_keys = seq_lens[t];
  } else {
    int lo = 0, hi = n_seqs - 1;          // last s with cu_q[s] <= t
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (cu_q[mid] <= t) lo = mid; else hi = mid - 1;
    }
    s = lo;
    n_keys = seq_lens[s] - (cu_q[s + 1] - 1 - t);
  }
  const bool active = h < heads;           // uniform per wave
  float* qs = smem + wid * W;
  if (active) {
    const T* qrow = q + (long)t * q_row_stride + (long)h * W;
    for (int i = lane; i < W; i += 64) qs[i] = IO<T>::ld(qrow + i) * scale;
  }
  __syncthreads();
  if (!active) return;

  const int* table = block_tables + (long)s * table_width;
  float m = -INFINITY, l = 0.f;
  float acc[LAT_MAX_ACC];
#pragma unroll
  for (int i = 0; i < LAT_MAX_ACC; ++i) acc[i] = 0.f;
  const int n_acc = (r + 63) >> 6;

  for (int k0 = 0; k0 < n_keys; k0 += 64) {
    const int key = k0 + lane;
    float sc = -INFINITY;
    if (key < n_keys) {
      const long blk = table[key / block_size];
      const T* krow = cache + (blk * block_size + key % block_size) * (long)W;
      float d = 0.f;
      for (int i = 0; i < W; ++i) d += qs[i] * IO<T>::ld(krow + i);
      sc = d;
    }
    const float m_new = fmaxf(m, wave_reduce_max(sc));
    const float alpha = __expf(m - m_new);       // m=-inf first: exp(-inf)=0
    const float p = (key < n_keys) ? __expf(sc - m_new) : 0.f;
    l = l * alpha + wave_reduce_sum(p);
    m = m_new;
#pragma unroll
    for (int i = 0; i < LAT_MAX_ACC; ++i) acc[i] *= alpha;
    const int nk = min(64, n_keys - k0);
    for (int j = 0; j < nk; ++j) {
      const float pj = __shfl(p, j, 64);
      const int kj = k0 + j;
      const long blk = table[kj / block_size];
      const T* vrow = cache + (blk * block_size + kj % block_size) * (long)W;
#pragma unroll
      for (int i = 0; i < LAT_MAX_ACC; ++i) {
        const int c = lane + 64 * i;
        if (i < n_acc && c < r) acc[i] += pj * IO<T>::ld(vrow + c);
      }
    }
  }
  const float inv = (l > 0.f) ? 1.0f / l : 0.f;
  float* orow = out + ((long)t * heads + h) * r;
#pragma unroll
  for (int i = 0; i < LAT_MAX_ACC; ++i) {
    const int c = lane + 64 * i;
    if (i < n_acc && c < r) orow[c] = acc[i] * inv;
  }
}

template <typename T>
void launch_latent_kv_store(T* cache, const T* dkv, const float* norm_w,
                            float eps, const long* pos,
                            const double* inv_freq, float mscale,
                            int rot_dims, const long* slots, int tokens,
                            int r, int rd, long dkv_stride, hipStream_t st) {
  if (tokens == 0) return;
  hipLaunchKernelGGL((latent_kv_store_kernel<T>), dim3(tokens), dim3(64), 0,
                     st, cache, dkv, norm_w, eps, pos, inv_freq, mscale,
                     rot_dims, slots, r, rd, dkv_stride);
}

template <typename T>
void launch_latent_attn(float* out, const T* q, const T* cache,
                        const int* block_tables, const int* cu_q,
                        const int* seq_lens, int tokens, int n_seqs,
                        int heads, int r, int rd, int block_size,
                        int table_width, float scale, long q_row_stride,
                        hipStream_t st) {
  if (tokens == 0) return;
  const int nw = heads < 4 ? heads : 4;
  const int W = r + rd;
  dim3 grid(tokens, (heads + nw - 1) / nw);
  hipLaunchKernelGGL((latent_attn_kernel<T>), grid, dim3(64 * nw),
                     (size_t)nw * W * sizeof(float), st, out, q, cache,
                     block_tables, cu_q, seq_lens, n_seqs, heads, r, rd,
                     block_size, table_width, scale, q_row_stride);
}

#define INST_LAT(T)                                                          \
  template void launch_latent_kv_store<T>(                                   \
      T*, const T*, const float*, float, const long*, const double*, float,  \
      int, const long*, int, int, int, long, hipStream_t);                   \
  template void launch_latent_attn<T>(float*, const T*, const T*,            \
                                      const int*, const int*, const int*,    \
                                      int, int, int, int, int, int, int,     \
                                      float, long, hipStream_t);
INST_LAT(float)
INST_LAT(unsigned short)

}  // namespace hyb
}  // namespace xllm
