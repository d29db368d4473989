// Decayed linear attention with a carried recurrent state.
//
//   S_t = decay_h * S_{t-1} + k_t v_t^T        (S is [D, Dv] per head, fp32)
//   o_t = S_t^T q_t
// with q, k, v = silu(projection), the activation fused here. The state
// lives in a slot pool [slots, H, D, Dv]; a sequence with ctx_len == 0 starts
// from zero whatever its slot held before.
//
// One workgroup per (sequence, head, 16-column slice of Dv): the columns of S
// are independent, so slices never talk to each other. Thread (j, r) owns the
// rows i = r, r+16, ... of column j; a token's output column is the sum over
// the 16 threads sharing j (a 16-lane shuffle reduction). Tokens are staged
// through LDS 16 at a time.
//
// Long prompt chunks run chunk-parallel: every `chunk` tokens first build
// their own state from zero (all chunks at once), a scan kernel turns these
// into the state before each chunk, and a second parallel pass produces the
// outputs. Same recurrence, re-associated only at chunk edges.
#include "hybrid_common.h"

namespace xllm {
namespace hyb {

constexpr int DA_VS = 16;      // value columns per workgroup
constexpr int DA_R = 16;       // row groups (threads per column)
constexpr int DA_TC = 16;      // tokens staged per LDS fill
constexpr int DA_MAXM = 16;    // D <= DA_R * DA_MAXM = 256

template <typename T>
__global__ void __launch_bounds__(256) decay_attn_kernel(
    float* __restrict__ out, const T* __restrict__ q, const T* __restrict__ k,
    const T* __restrict__ v, const float* __restrict__ decay,
    float* __restrict__ state, const int* __restrict__ slots,
    const int* __restrict__ cu_q, const int* __restrict__ ctx_lens, int heads,
    int D, int Dv, long q_stride, long k_stride, long v_stride, int mode,
    int chunk, int max_chunks, float* __restrict__ ws) {
  extern __shared__ float smem[];
  float* qs = smem;                       // [TC][D]
  float* ks = qs + DA_TC * D;             // [TC][D]
  float* vs = ks + DA_TC * D;             // [TC][VS]

  // mode 0: whole sequence chunk in one workgroup (state slot in and out).
  // mode 1: tokens [c*chunk, (c+1)*chunk) from a zero state, no outputs;
  //         the chunk's own state goes to ws[s*max_chunks + c].
  // mode 2: the same tokens starting from ws[s*max_chunks + c] (filled by
  //         the scan kernel below), outputs written, no state out.
  const int s = blockIdx.x / max_chunks, cidx = blockIdx.x % max_chunks;
  const int h = blockIdx.y, v0 = blockIdx.z * DA_VS;
  const int tid = threadIdx.x;
  const int j = tid / DA_R, r = tid % DA_R;
  const int col = v0 + j;
  const bool col_ok = col < Dv;
  int t0 = cu_q ? cu_q[s] : s;
  int t1 = cu_q ? cu_q[s + 1] : s + 1;
  if (mode != 0) {
    t0 += cidx * chunk;
    if (t0 >= t1) return;                   // uniform for the workgroup
    t1 = min(t1, t0 + chunk);
  }
  const int slot = slots[s];
  const float dec = decay[h];
  const int M = (D + DA_R - 1) / DA_R;

  float S[DA_MAXM];
#pragma unroll
  for (int m = 0; m < DA_MAXM; ++m) S[m] = 0.f;
  float* sp = (slot >= 0)
      ? state + (((long)slot * heads + h) * D) * (long)Dv : nullptr;
  bool load = sp && ctx_lens[s] > 0;
  if (mode != 0) {
    sp = ws + ((((long)s * max_chunks + cidx) * heads + h) * D) * (long)Dv;
    load = mode == 2;
  }
  // The 16-column slice of the state is 64 B per row: move it with float4
  // accesses (a wave covers 16 whole rows) through an LDS tile instead of
  // one 4 B element per lane and row.
  float* tile = smem;                     // [D][DA_VS + 1], reused by staging
  const bool vec_ok = (Dv % 4 == 0) && (v0 + DA_VS <= Dv);
  if (load) {
    if (vec_ok) {
      for (int idx = tid; idx < D * 4; idx += 256) {
        const int i = idx >> 2, c4 = (idx & 3) * 4;
        const float4 x = *reinterpret_cast<const float4*>(
            sp + (long)i * Dv + v0 + c4);
        float* d = tile + i * (DA_VS + 1) + c4;
        d[0] = x.x; d[1] = x.y; d[2] = x.z; d[3] = x.w;
      }
      __syncthreads();
#pragma unroll
      for (int m = 0; m < DA_MAXM; ++m) {
        const int i = r + DA_R * m;
        if (m < M && i < D) S[m] = tile[i * (DA_VS + 1) + j];
      }
    } else if (col_ok) {
#pragma unroll
      for (int m = 0; m < DA_MAXM; ++m) {
        const int i = r + DA_R * m;
        if (m < M && i < D) S[m] = sp[(long)i * Dv + col];
      }
    }
  }

  for (int tb = t0; tb < t1; tb += DA_TC) {
    const int nt = min(DA_TC, t1 - tb);
    __syncthreads();                      // previous tile fully consumed
    for (int idx = tid; idx < nt * D; idx += 256) {
      const int tt = idx / D, i = idx - tt * D;
      const long row = tb + tt;
      qs[idx] = IO<T>::rnd(siluf_(IO<T>::ld(q + row * q_stride + h * D + i)));
      ks[idx] = IO<T>::rnd(siluf_(IO<T>::ld(k + row * k_stride + h * D + i)));
    }
    for (int idx = tid; idx < nt * DA_VS; idx += 256) {
      const int tt = idx / DA_VS, jj = idx - tt * DA_VS;
      const long row = tb + tt;
      vs[idx] = (v0 + jj < Dv)
          ? IO<T>::rnd(siluf_(IO<T>::ld(v + row * v_stride + h * Dv + v0 + jj)))
          : 0.f;
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float vj = vs[tt * DA_VS + j];
      float o = 0.f;
#pragma unroll
      for (int m = 0; m < DA_MAXM; ++m) {
        const int i = r + DA_R * m;
        if (m < M && i < D) {
          S[m] = dec * S[m] + ks[tt * D + i] * vj;
          o += S[m] * qs[tt * D + i];
        }
      }
      if (mode != 1) {
        o = group_reduce_sum<DA_R>(o);
        if (r == 0 && col_ok)
          out[((long)(tb + tt) * heads + h) * Dv + col] = o;
      }
    }
  }
  if (sp && mode != 2) {
    if (vec_ok) {
      __syncthreads();                    // staging buffers are done with
#pragma unroll
      for (int m = 0; m < DA_MAXM; ++m) {
        const int i = r + DA_R * m;
        if (m < M && i < D) tile[i * (DA_VS + 1) + j] = S[m];
      }
      __syncthreads();
      for (int idx = tid; idx < D * 4; idx += 256) {
        const int i = idx >> 2, c4 = (idx & 3) * 4;
        const float* d = tile + i * (DA_VS + 1) + c4;
        *reinterpret_cast<float4*>(sp + (long)i * Dv + v0 + c4) =
            make_float4(d[0], d[1], d[2], d[3]);
      }
    } else if (col_ok) {
#pragma unroll
      for (int m = 0; m < DA_MAXM; ++m) {
        const int i = r + DA_R * m;
        if (m < M && i < D) sp[(long)i * Dv + col] = S[m];
      }
    }
  }
}

// Decode (one token per sequence): the step is a pure stream over the state,
// so one workgroup takes a whole (sequence, head) state and moves it as
// full rows: thread (rg, tc) owns columns 4*tc..4*tc+3 of rows rg, rg+RG, ...
// (float4 per row; a wave covers whole 512 B rows at Dv = 128). Partial
// outputs of the RG row groups are summed through LDS.
template <typename T>
__global__ void __launch_bounds__(256) decay_attn_decode_kernel(
    float* __restrict__ out, const T* __restrict__ q, const T* __restrict__ k,
    const T* __restrict__ v, const float* __restrict__ decay,
    float* __restrict__ state, const int* __restrict__ slots,
    const int* __restrict__ ctx_lens, int heads, int D, int Dv, long q_stride,
    long k_stride, long v_stride) {
  extern __shared__ float smem[];
  const int Dp = (D + 3) & ~3;      // keeps the float4 regions 16 B aligned
  float* qs = smem;                 // [Dp]
  float* ks = qs + Dp;              // [Dp]
  float* vs = ks + Dp;              // [Dv]
  float* part = vs + Dv;            // [RG][Dv]
  const int s = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int TCn = Dv >> 2, RG = 256 / TCn;
  const int rg = tid / TCn, tc = tid - rg * TCn;
  for (int i = tid; i < D; i += 256) {
    qs[i] = IO<T>::rnd(siluf_(IO<T>::ld(q + s * q_stride + h * D + i)));
    ks[i] = IO<T>::rnd(siluf_(IO<T>::ld(k + s * k_stride + h * D + i)));
  }
  for (int i = tid; i < Dv; i += 256)
    vs[i] = IO<T>::rnd(siluf_(IO<T>::ld(v + s * v_stride + h * Dv + i)));
  __syncthreads();
  const int slot = slots[s];
  const bool load = slot >= 0 && ctx_lens[s] > 0;
  const float a = decay[h];
  float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
  if (rg < RG) {
    float* sp = state + (((long)max(slot, 0) * heads + h) * D) * (long)Dv + 4 * tc;
    const float4 vv = *reinterpret_cast<const float4*>(vs + 4 * tc);
    for (int i = rg; i < D; i += RG) {
      float4 S = make_float4(0.f, 0.f, 0.f, 0.f);
      if (load) S = *reinterpret_cast<const float4*>(sp + (long)i * Dv);
      const float ki = ks[i], qi = qs[i];
      S.x = a * S.x + ki * vv.x; S.y = a * S.y + ki * vv.y;
      S.z = a * S.z + ki * vv.z; S.w = a * S.w + ki * vv.w;
      o.x += S.x * qi; o.y += S.y * qi; o.z += S.z * qi; o.w += S.w * qi;
      if (slot >= 0) *reinterpret_cast<float4*>(sp + (long)i * Dv) = S;
    }
    *reinterpret_cast<float4*>(part + rg * Dv + 4 * tc) = o;
  }
  __syncthreads();
  for (int c = tid; c < Dv; c += 256) {
    float acc = 0.f;
    for (int g2 = 0; g2 < RG; ++g2) acc += part[g2 * Dv + c];
    out[((long)s * heads + h) * Dv + c] = acc;
  }
}

// Sequential pass over a sequence's chunk states (one thread per state
// element): ws[c] <- state before chunk c; the state after the last chunk
// goes to the sequence's slot.
__global__ void decay_scan_kernel(float* __restrict__ ws,
                                  float* __restrict__ state,
                                  const float* __restrict__ decay,
                                  const int* __restrict__ slots,
                                  const int* __restrict__ cu_q,
                                  const int* __restrict__ ctx_lens, int heads,
                                  long per_head, int chunk, int max_chunks) {
  const int s = blockIdx.y;
  const long per_seq = per_head * heads;
  const long e = blockIdx.x * (long)blockDim.x + threadIdx.x;
  if (e >= per_seq) return;
  const int h = (int)(e / per_head);
  const int qlen = cu_q[s + 1] - cu_q[s];
  const int n_chunks = (qlen + chunk - 1) / chunk;
  const int slot = slots[s];
  const float a = decay[h];
  float S = (slot >= 0 && ctx_lens[s] > 0) ? state[slot * per_seq + e] : 0.f;
  const float a_full = powf(a, (float)chunk);
  for (int c = 0; c < n_chunks; ++c) {
    float* w = ws + ((long)s * max_chunks + c) * per_seq + e;
    const float local = *w;
    *w = S;
    const int len = min(chunk, qlen - c * chunk);
    S = (len == chunk ? a_full : powf(a, (float)len)) * S + local;
  }
  if (slot >= 0) state[slot * per_seq + e] = S;
}

template <typename T>
void launch_decay_attn(float* out, const T* q, const T* k, const T* v,
                       const float* decay, float* state, const int* slots,
                       const int* cu_q, const int* ctx_lens, int n_seqs,
                       int heads, int D, int Dv, long q_stride, long k_stride,
                       long v_stride, int chunk, int max_chunks, float* ws,
                       hipStream_t st) {
  if (n_seqs == 0) return;
  const size_t lds = (size_t)(2 * DA_TC * D + DA_TC * DA_VS) * sizeof(float);
  const int vz = (Dv + DA_VS - 1) / DA_VS;
  if (cu_q == nullptr && Dv % 4 == 0 && Dv <= 1024) {
    const int RG = 256 / (Dv / 4);
    const size_t l2 = (size_t)(2 * ((D + 3) & ~3) + Dv + RG * Dv) * sizeof(float);
    if (l2 <= 64 * 1024) {
      hipLaunchKernelGGL((decay_attn_decode_kernel<T>), dim3(n_seqs, heads),
                         dim3(256), l2, st, out, q, k, v, decay, state, slots,
                         ctx_lens, heads, D, Dv, q_stride, k_stride, v_stride);
      return;
    }
  }
  if (ws == nullptr || max_chunks <= 1) {
    hipLaunchKernelGGL((decay_attn_kernel<T>), dim3(n_seqs, heads, vz),
                       dim3(256), lds, st, out, q, k, v, decay, state, slots,
                       cu_q, ctx_lens, heads, D, Dv, q_stride, k_stride,
                       v_stride, 0, 0, 1, nullptr);
    return;
  }
  // chunk-parallel: local chunk states, a short scan, then the outputs
  dim3 grid(n_seqs * max_chunks, heads, vz);
  hipLaunchKernelGGL((decay_attn_kernel<T>), grid, dim3(256), lds, st, out, q,
                     k, v, decay, state, slots, cu_q, ctx_lens, heads, D, Dv,
                     q_stride, k_stride, v_stride, 1, chunk, max_chunks, ws);
  const long per_head = (long)D * Dv;
  const long per_seq = per_head * heads;
  hipLaunchKernelGGL(decay_scan_kernel,
                     dim3((unsigned)((per_seq + 255) / 256), n_seqs),
                     dim3(256), 0, st, ws, state, decay, slots, cu_q,
                     ctx_lens, heads, per_head, chunk, max_chunks);
  hipLaunchKernelGGL((decay_attn_kernel<T>), grid, dim3(256), lds, st, out, q,
                     k, v, decay, state, slots, cu_q, ctx_lens, heads, D, Dv,
                     q_stride, k_stride, v_stride, 2, chunk, max_chunks, ws);
}

#define INST_DA(T)                                                            \
  template void launch_decay_attn<T>(                                         \
      float*, const T*, const T*, const T*, const float*, float*, const int*, \
      const int*, const int*, int, int, int, int, long, long, long, int, int, \
      float*, hipStream_t);
INST_DA(float)
INST_DA(unsigned short)

}  // namespace hyb
}  // namespace xllm
