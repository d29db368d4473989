// Short causal convolution over time, one filter per channel, with the last
// taps-1 inputs of every sequence carried in a slot pool.
//
//   y[t, c] = act( sum_j w[c, j] * u[t - taps + 1 + j, c] + b[c] )
//
// u before the start of the sequence is zero; u before the start of this
// step's tokens comes from the sequence's state rows (state[slot, i] holds the
// input of position ctx - (taps-1) + i). Reads are guarded by position, so a
// reused slot never has to be cleared.
//
// The channels are seen as heads of `hd` channels; a thread owns the pair
// (2j, 2j+1) of one head so that an interleaved rotary turn of the first
// `rot_dims` channels of each head can follow in registers. The result goes
// to a row-major tensor or straight into a paged cache
// [blocks, heads, block, hd] at the token's slot.
//
// A second kernel moves the state forward once every reader of the old state
// has been launched (same stream).
#include "hybrid_common.h"

namespace xllm {
namespace hyb {

constexpr int SC_MAX_TAPS = 16;

XLLM_DEV int seq_of_token(const int* __restrict__ cu_q, int n_seqs, int t) {
  int lo = 0, hi = n_seqs - 1;             // last s with cu_q[s] <= t
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (cu_q[mid] <= t) lo = mid; else hi = mid - 1;
  }
  return lo;
}

// TAPS > 0: the filter length is a compile-time constant, the filter and a
// sliding window of the last inputs stay in registers, and every token of the
// tile costs one new input load. TAPS == 0: any length, every tap loaded.
template <typename T, int TAPS>
__global__ void __launch_bounds__(256) short_conv_kernel(
    T* __restrict__ out, long out_stride, T* __restrict__ cache,
    const long* __restrict__ slot_mapping, int block_size,
    const T* __restrict__ x, long x_stride, const T* __restrict__ w,
    const T* __restrict__ bias, const T* __restrict__ state, long state_row,
    int state_off, const int* __restrict__ slots, const int* __restrict__ cu_q,
    const int* __restrict__ ctx_lens, int n_seqs, int heads, int hd, int taps,
    int act_silu, int rot_dims, const long* __restrict__ pos,
    const double* __restrict__ inv_freq, int tokens, int tile) {
  const int ppairs = (hd + 1) >> 1;
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= heads * ppairs) return;
  const int h = idx / ppairs, j = idx - h * ppairs;
  const int d0 = 2 * j;
  const int c0 = h * hd + d0;
  const bool two = d0 + 1 < hd;
  const int K1 = taps - 1;
  const float b0 = bias ? IO<T>::ld(bias + c0) : 0.f;
  const float b1 = (bias && two) ? IO<T>::ld(bias + c0 + 1) : 0.f;
  constexpr int NT = TAPS > 0 ? TAPS : 1;
  float w0[NT], w1[NT], h0[NT], h1[NT];    // filter and window (TAPS > 0)
  if (TAPS > 0) {
#pragma unroll
    for (int jj = 0; jj < NT; ++jj) {
      w0[jj] = IO<T>::ld(w + (long)c0 * taps + jj);
      w1[jj] = two ? IO<T>::ld(w + (long)(c0 + 1) * taps + jj) : 0.f;
      h0[jj] = h1[jj] = 0.f;
    }
  }

  // a workgroup walks `tile` consecutive tokens: the sequence lookup is done
  // once and then only moved forward
  const int t_first = blockIdx.y * tile;
  const int t_last = min(t_first + tile, tokens);
  int s = cu_q ? seq_of_token(cu_q, n_seqs, t_first) : t_first;
  for (int t = t_first; t < t_last; ++t) {
    int t0;
    if (cu_q) {
      while (s + 1 < n_seqs && t >= cu_q[s + 1]) ++s;
      t0 = cu_q[s];
    } else {
      s = t; t0 = t;
    }
    const int li = t - t0;
    const int p = ctx_lens[s] + li;        // position of this token
    const int slot = slots[s];
    // input of tap jj (position p - K1 + jj), zero before the sequence
    auto tap = [&](int jj, float& u0, float& u1) {
      u0 = u1 = 0.f;
      const int src = li - K1 + jj;        // local index among this step's rows
      if (p - K1 + jj < 0) return;
      const T* row;
      if (src >= 0) {
        row = x + (long)(t0 + src) * x_stride + c0;
      } else {
        if (slot < 0) return;
        row = state + ((long)slot * K1 + (K1 + src)) * state_row + state_off + c0;
      }
      u0 = IO<T>::ld(row);
      if (two) u1 = IO<T>::ld(row + 1);
    };
    float a0 = b0, a1 = b1;
    if (TAPS > 0) {
      if (t == t_first || li == 0) {       // (re)fill the window
#pragma unroll
        for (int jj = 0; jj < NT - 1; ++jj) tap(jj, h0[jj], h1[jj]);
      } else {
#pragma unroll
        for (int jj = 0; jj < NT - 1; ++jj) { h0[jj] = h0[jj + 1]; h1[jj] = h1[jj + 1]; }
      }
      tap(NT - 1, h0[NT - 1], h1[NT - 1]);
#pragma unroll
      for (int jj = 0; jj < NT; ++jj) { a0 += w0[jj] * h0[jj]; a1 += w1[jj] * h1[jj]; }
    } else {
      for (int jj = 0; jj < taps; ++jj) {
        float u0, u1;
        tap(jj, u0, u1);
        a0 += IO<T>::ld(w + (long)c0 * taps + jj) * u0;
        if (two) a1 += IO<T>::ld(w + (long)(c0 + 1) * taps + jj) * u1;
      }
    }
    if (act_silu) { a0 = siluf_(a0); a1 = siluf_(a1); }
    if (two && d0 + 1 < rot_dims) {
      double sn, cs;
      sincos((double)pos[t] * inv_freq[j], &sn, &cs);
      const float cf = (float)cs, sf = (float)sn;
      const float u = a0, v = a1;
      a0 = u * cf - v * sf;
      a1 = v * cf + u * sf;
    }
    T* dst;
    if (cache) {
      const long sl = slot_mapping[t];
      if (sl < 0) continue;
      const long blk = sl / block_size, off = sl % block_size;
      dst = cache + ((blk * heads + h) * block_size + off) * (long)hd + d0;
    } else {
      dst = out + (long)t * out_stride + c0;
    }
    IO<T>::st(dst, a0);
    if (two) IO<T>::st(dst + 1, a1);
  }
}

// state[slot, i] <- input of position (ctx + len) - (taps-1) + i, from this
// step's rows or, for a step shorter than the state, from the old state.
// Ascending i only ever reads old entries above the one being written.
template <typename T>
__global__ void short_conv_state_kernel(
    T* __restrict__ state, long state_row, const T* __restrict__ x,
    long x_stride, const int* __restrict__ slots,
    const int* __restrict__ cu_q, int channels, int taps) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int slot = slots[s];
  if (slot < 0) return;
  const int t0 = cu_q ? cu_q[s] : s;
  const int len = cu_q ? cu_q[s + 1] - t0 : 1;
  const int K1 = taps - 1;
  T* st = state + (long)slot * K1 * state_row + c;
  for (int i = 0; i < K1; ++i) {
    const int local = len - K1 + i;
    if (local >= 0) st[(long)i * state_row] = x[(long)(t0 + local) * x_stride + c];
    else st[(long)i * state_row] = st[(long)(i + len) * state_row];
  }
}

template <typename T>
void launch_short_conv(T* out, long out_stride, T* cache,
                       const long* slot_mapping, int block_size, const T* x,
                       long x_stride, const T* w, const T* bias,
                       const T* state, long state_row, int state_off,
                       const int* slots, const int* cu_q, const int* ctx_lens,
                       int tokens, int n_seqs, int heads, int hd, int taps,
                       int act_silu, int rot_dims, const long* pos,
                       const double* inv_freq, hipStream_t st) {
  if (tokens == 0 || heads * hd == 0) return;
  const int n = heads * ((hd + 1) / 2);
  const int bx = n >= 256 ? 256 : ((n + 63) / 64) * 64;
  // long batches: 16 tokens per workgroup (one input load per token);
  // short ones (decode) keep every token in a workgroup of its own
  const int tile = tokens >= 2048 ? 16 : tokens >= 256 ? 4 : 1;
  dim3 grid((n + bx - 1) / bx, (tokens + tile - 1) / tile);
#define SC_LAUNCH(TAPS)                                                       \
  hipLaunchKernelGGL((short_conv_kernel<T, TAPS>), grid, dim3(bx), 0, st, out, \
                     out_stride, cache, slot_mapping, block_size, x, x_stride, \
                     w, bias, state, state_row, state_off, slots, cu_q,       \
                     ctx_lens, n_seqs, heads, hd, taps, act_silu, rot_dims,   \
                     pos, inv_freq, tokens, tile)
  switch (taps) {
    case 2: SC_LAUNCH(2); break;
    case 3: SC_LAUNCH(3); break;
    case 4: SC_LAUNCH(4); break;
    default: SC_LAUNCH(0); break;
  }
#undef SC_LAUNCH
}

template <typename T>
void launch_short_conv_state(T* state, long state_row, const T* x,
                             long x_stride, const int* slots, const int* cu_q,
                             int n_seqs, int channels, int taps,
                             hipStream_t st) {
  if (n_seqs == 0 || channels == 0 || taps <= 1) return;
  dim3 grid((channels + 255) / 256, n_seqs);
  hipLaunchKernelGGL((short_conv_state_kernel<T>), grid, dim3(256), 0, st,
                     state, state_row, x, x_stride, slots, cu_q, channels,
                     taps);
}

#define INST_SC(T)                                                            \
  template void launch_short_conv<T>(                                         \
      T*, long, T*, const long*, int, const T*, long, const T*, const T*,     \
      const T*, long, int, const int*, const int*, const int*, int, int, int, \
      int, int, int, int, const long*, const double*, hipStream_t);           \
  template void launch_short_conv_state<T>(T*, long, const T*, long,          \
                                           const int*, const int*, int, int,  \
                                           int, hipStream_t);
INST_SC(float)
INST_SC(unsigned short)

}  // namespace hyb
}  // namespace xllm
