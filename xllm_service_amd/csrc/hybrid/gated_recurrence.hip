// Linear recurrence with a data-dependent decay and a carried fp32 state:
//
//   S_t = diag(a_t) S_{t-1} + k_t v_t^T        (S is [D, Dv] per head)
//   o_t = S_t^T q_t (+ skip_h * v_t)
//
// Two ways of making a_t, k_t, q_t from the projections, fused into the
// staging loads (everything below is fp32; only the loads convert):
//
//   GR_SSM  selective state space: dt = softplus(dt_raw + dt_bias_h),
//           a_t = exp(-exp(A_log_h) dt) (one scalar per head), k_t = dt B_t,
//           q_t = C_t, v_t = x_t, skip = D_h. B and C are shared by the heads
//           of a group.
//   GR_GLA  gated linear attention: a_t[i] = sigmoid(z_t[i] + zb[i])^(1/tau)
//           per key channel, q_t scaled by a constant.
//
// The state lives in a slot pool [slots, H, D, Dv]; a sequence with
// ctx_len == 0 starts from zero whatever its slot held before; slot < 0 runs
// from zero and stores nothing.
//
// Prompt chunks: one workgroup per (sequence, head, 16*CPT columns of Dv);
// thread (j, r) owns rows r, r+16, ... of CPT neighbouring columns (CPT = 4
// for wide values: a key/query/decay value read from LDS then feeds 8 FMAs);
// a 16-lane DPP reduction sums a token's output. Long chunks run piece-parallel: every piece builds its own state
// from zero together with the product of its decays, a scan turns these into
// the state before each piece, a second pass writes the outputs. Decode: one
// workgroup per (sequence, head) streams the state as whole rows.
#include <cstdlib>

#include "hybrid_common.h"

namespace xllm {
namespace hyb {

constexpr int GR_SSM = 0;
constexpr int GR_GLA = 1;
constexpr int GR_CG = 16;      // column groups per workgroup
constexpr int GR_R = 16;       // row groups (threads per column group)
constexpr int GR_TC = 16;      // tokens staged per LDS fill
constexpr int GR_MAXM = 16;    // D <= GR_R * GR_MAXM = 256

// Sum over the 16 lanes of a DPP row, left in every lane: lane-crossing
// inside the vector ALU (quad permutes, then the two mirror modes) instead of
// four trips through the LDS crossbar.
XLLM_DEV float row16_sum(float v) {
  v += __int_as_float(__builtin_amdgcn_update_dpp(
      0, __float_as_int(v), 0xB1, 0xF, 0xF, true));    // quad_perm [1,0,3,2]
  v += __int_as_float(__builtin_amdgcn_update_dpp(
      0, __float_as_int(v), 0x4E, 0xF, 0xF, true));    // quad_perm [2,3,0,1]
  v += __int_as_float(__builtin_amdgcn_update_dpp(
      0, __float_as_int(v), 0x141, 0xF, 0xF, true));   // row_half_mirror
  v += __int_as_float(__builtin_amdgcn_update_dpp(
      0, __float_as_int(v), 0x140, 0xF, 0xF, true));   // row_mirror
  return v;
}

XLLM_DEV float softplusf_(float x) {
  return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x)));
}

template <typename T>
struct GRArgs {
  const T* q; const T* k; const T* v; const T* g;
  long q_stride, k_stride, v_stride, g_stride;
  const float* p0; const float* p1; const float* p2;
  float c0, c1;
  int heads, groups, D, Dv;
};

// stage one token's q, k (scaled), decay for head h into LDS rows
template <typename T, int KIND>
XLLM_DEV void gr_stage_row(const GRArgs<T>& A, long row, int h, int i,
                           float dt, float* qd, float* kd, float* ad) {
  const int kg = h / (A.heads / A.groups);
  const float qv = IO<T>::ld(A.q + row * A.q_stride + kg * A.D + i);
  const float kv = IO<T>::ld(A.k + row * A.k_stride + kg * A.D + i);
  if (KIND == GR_SSM) {
    *qd = qv;
    *kd = dt * kv;
  } else {
    *qd = qv * A.c1;
    *kd = kv;
    const float z = IO<T>::ld(A.g + row * A.g_stride + h * A.D + i)
                    + A.p0[h * A.D + i];
    *ad = expf(-softplusf_(-z) * A.c0);
  }
}

template <typename T, int KIND, int CPT>
__global__ void __launch_bounds__(256) gated_recurrence_kernel(
    float* __restrict__ out, GRArgs<T> A, float* __restrict__ state,
    const int* __restrict__ slots, const int* __restrict__ cu_q,
    const int* __restrict__ ctx_lens, int mode, int chunk, int max_chunks,
    float* __restrict__ ws, float* __restrict__ wa) {
  extern __shared__ float smem[];
  constexpr int VS = GR_CG * CPT;         // value columns per workgroup
  const int D = A.D, Dv = A.Dv, heads = A.heads;
  const int Dd = (KIND == GR_SSM) ? 1 : D;
  float* qs = smem;                       // [TC][D]
  float* ks = qs + GR_TC * D;             // [TC][D]
  float* as = ks + GR_TC * D;             // [TC][Dd] (SSM: [TC] a, [TC] dt)
  float* vs = as + GR_TC * (KIND == GR_SSM ? 2 : D);   // [TC][VS]

  // mode 0: the whole chunk of a sequence in one workgroup (slot in and out)
  // mode 1: tokens [c*chunk, (c+1)*chunk) from a zero state, no outputs; the
  //         piece's own state goes to ws[s*max_chunks + c] and the product of
  //         its decays to wa[s*max_chunks + c]
  // mode 2: the same tokens starting from ws[s*max_chunks + c] (as the scan
  //         left it), outputs written, no state out
  const int s = blockIdx.x / max_chunks, cidx = blockIdx.x % max_chunks;
  const int h = blockIdx.y, v0 = blockIdx.z * VS;
  const int tid = threadIdx.x;
  const int j = tid / GR_R, r = tid % GR_R;
  const int col = v0 + j * CPT;           // first of this thread's columns
  int t0 = cu_q ? cu_q[s] : s;
  int t1 = cu_q ? cu_q[s + 1] : s + 1;
  if (mode != 0) {
    t0 += cidx * chunk;
    if (t0 >= t1) return;                 // uniform for the workgroup
    t1 = min(t1, t0 + chunk);
  }
  const int slot = slots[s];
  const int M = (D + GR_R - 1) / GR_R;

  float S[GR_MAXM][CPT], P[GR_MAXM];
#pragma unroll
  for (int m = 0; m < GR_MAXM; ++m) {
    P[m] = 1.f;
#pragma unroll
    for (int c = 0; c < CPT; ++c) S[m][c] = 0.f;
  }
  float* sp = (slot >= 0)
      ? state + (((long)slot * heads + h) * D) * (long)Dv : nullptr;
  bool load = sp && ctx_lens[s] > 0;
  if (mode != 0) {
    sp = ws + ((((long)s * max_chunks + cidx) * heads + h) * D) * (long)Dv;
    load = mode == 2;
  }
  const bool vec = CPT == 4 && (Dv & 3) == 0 && col + 3 < Dv;
  if (load) {
#pragma unroll
    for (int m = 0; m < GR_MAXM; ++m) {
      const int i = r + GR_R * m;
      if (m < M && i < D) {
        if (vec) {
          const float4 x = *reinterpret_cast<const float4*>(
              sp + (long)i * Dv + col);
          S[m][0] = x.x; S[m][CPT > 1 ? 1 : 0] = x.y;
          S[m][CPT > 2 ? 2 : 0] = x.z; S[m][CPT > 3 ? 3 : 0] = x.w;
        } else {
#pragma unroll
          for (int c = 0; c < CPT; ++c)
            if (col + c < Dv) S[m][c] = sp[(long)i * Dv + col + c];
        }
      }
    }
  }
  float dt_bias = 0.f, negA = 0.f, skip = 0.f;
  if (KIND == GR_SSM) {
    dt_bias = A.p0[h];
    negA = -expf(A.p1[h]);
    skip = A.p2 ? A.p2[h] : 0.f;
  }

  for (int tb = t0; tb < t1; tb += GR_TC) {
    const int nt = min(GR_TC, t1 - tb);
    __syncthreads();                      // previous tile fully consumed
    if (KIND == GR_SSM) {
      if (tid < nt) {
        const float dt = softplusf_(
            IO<T>::ld(A.g + (long)(tb + tid) * A.g_stride + h) + dt_bias);
        as[tid] = expf(negA * dt);
        as[GR_TC + tid] = dt;
      }
      __syncthreads();
    }
    for (int idx = tid; idx < nt * D; idx += 256) {
      const int tt = idx / D, i = idx - tt * D;
      const long row = tb + tt;
      const float dt = (KIND == GR_SSM) ? as[GR_TC + tt] : 0.f;
      gr_stage_row<T, KIND>(A, row, h, i, dt, qs + idx, ks + idx,
                            as + (KIND == GR_SSM ? 0 : idx));
    }
    for (int idx = tid; idx < nt * VS; idx += 256) {
      const int tt = idx / VS, jj = idx - tt * VS;
      const long row = tb + tt;
      vs[idx] = (v0 + jj < Dv)
          ? IO<T>::ld(A.v + row * A.v_stride + h * Dv + v0 + jj) : 0.f;
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      float vj[CPT], o[CPT];
#pragma unroll
      for (int c = 0; c < CPT; ++c) {
        vj[c] = vs[tt * VS + j * CPT + c];
        o[c] = 0.f;
      }
#pragma unroll
      for (int m = 0; m < GR_MAXM; ++m) {
        const int i = r + GR_R * m;
        if (m < M && i < D) {
          const float a = (KIND == GR_SSM) ? as[tt] : as[tt * D + i];
          const float kk = ks[tt * D + i], qq = qs[tt * D + i];
#pragma unroll
          for (int c = 0; c < CPT; ++c) {
            S[m][c] = a * S[m][c] + kk * vj[c];
            o[c] += S[m][c] * qq;
          }
          if (mode == 1) P[m] *= a;
        }
      }
      if (mode != 1) {
#pragma unroll
        for (int c = 0; c < CPT; ++c) o[c] = row16_sum(o[c]);
        if (r == 0) {
          float* op = out + ((long)(tb + tt) * heads + h) * Dv + col;
#pragma unroll
          for (int c = 0; c < CPT; ++c)
            if (col + c < Dv) op[c] = o[c] + skip * vj[c];
        }
      }
    }
  }
  if (sp && mode != 2) {
#pragma unroll
    for (int m = 0; m < GR_MAXM; ++m) {
      const int i = r + GR_R * m;
      if (m < M && i < D) {
        if (vec) {
          *reinterpret_cast<float4*>(sp + (long)i * Dv + col) = make_float4(
              S[m][0], S[m][CPT > 1 ? 1 : 0], S[m][CPT > 2 ? 2 : 0],
              S[m][CPT > 3 ? 3 : 0]);
        } else {
#pragma unroll
          for (int c = 0; c < CPT; ++c)
            if (col + c < Dv) sp[(long)i * Dv + col + c] = S[m][c];
        }
      }
    }
  }
  if (mode == 1 && j == 0 && v0 == 0) {
    float* ap = wa + (((long)s * max_chunks + cidx) * heads + h) * (long)Dd;
#pragma unroll
    for (int m = 0; m < GR_MAXM; ++m) {
      const int i = r + GR_R * m;
      if (m < M && i < Dd) ap[i] = P[m];
    }
  }
}

// Sequential pass over a sequence's piece states (one thread per state
// element): ws[c] <- state before piece c; the state after the last piece
// goes to the sequence's slot.
__global__ void gated_recurrence_scan_kernel(
    float* __restrict__ ws, const float* __restrict__ wa,
    float* __restrict__ state, const int* __restrict__ slots,
    const int* __restrict__ cu_q, const int* __restrict__ ctx_lens, int heads,
    int D, int Dv, int Dd, int chunk, int max_chunks) {
  const int s = blockIdx.y;
  const long per_head = (long)D * Dv;
  const long per_seq = per_head * heads;
  const long e = blockIdx.x * (long)blockDim.x + threadIdx.x;
  if (e >= per_seq) return;
  const int h = (int)(e / per_head);
  const int i = (int)((e - h * per_head) / Dv);
  const int qlen = cu_q[s + 1] - cu_q[s];
  const int n_chunks = (qlen + chunk - 1) / chunk;
  const int slot = slots[s];
  float S = (slot >= 0 && ctx_lens[s] > 0) ? state[slot * per_seq + e] : 0.f;
  for (int c = 0; c < n_chunks; ++c) {
    const long pc = (long)s * max_chunks + c;
    float* w = ws + pc * per_seq + e;
    const float local = *w;
    *w = S;
    S = wa[(pc * heads + h) * Dd + (Dd == 1 ? 0 : i)] * S + local;
  }
  if (slot >= 0) state[slot * per_seq + e] = S;
}

// Decode (one token per sequence): thread (rg, tc) owns columns 4tc..4tc+3 of
// rows rg, rg+RG, ... (float4 per row); partial outputs of the RG row groups
// are summed through LDS.
template <typename T, int KIND>
__global__ void __launch_bounds__(256) gated_recurrence_decode_kernel(
    float* __restrict__ out, GRArgs<T> A, float* __restrict__ state,
    const int* __restrict__ slots, const int* __restrict__ ctx_lens) {
  extern __shared__ float smem[];
  const int D = A.D, Dv = A.Dv, heads = A.heads;
  const int Dp = (D + 3) & ~3;      // keeps the float4 regions 16 B aligned
  float* qs = smem;                 // [Dp]
  float* ks = qs + Dp;              // [Dp]
  float* as = ks + Dp;              // [Dp]
  float* vs = as + Dp;              // [Dv]
  float* part = vs + Dv;            // [RG][Dv]
  const int s = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int TCn = Dv >> 2, RG = 256 / TCn;
  const int rg = tid / TCn, tc = tid - rg * TCn;
  float dt = 0.f, skip = 0.f, a_sc = 1.f;
  if (KIND == GR_SSM) {
    dt = softplusf_(IO<T>::ld(A.g + s * A.g_stride + h) + A.p0[h]);
    a_sc = expf(-expf(A.p1[h]) * dt);
    skip = A.p2 ? A.p2[h] : 0.f;
  }
  for (int i = tid; i < D; i += 256)
    gr_stage_row<T, KIND>(A, s, h, i, dt, qs + i, ks + i, as + i);
  for (int i = tid; i < Dv; i += 256)
    vs[i] = IO<T>::ld(A.v + s * A.v_stride + h * Dv + i);
  __syncthreads();
  const int slot = slots[s];
  const bool load = slot >= 0 && ctx_lens[s] > 0;
  float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
  if (rg < RG) {
    float* sp = state + (((long)max(slot, 0) * heads + h) * D) * (long)Dv + 4 * tc;
    const float4 vv = *reinterpret_cast<const float4*>(vs + 4 * tc);
    for (int i = rg; i < D; i += RG) {
      float4 S = make_float4(0.f, 0.f, 0.f, 0.f);
      if (load) S = *reinterpret_cast<const float4*>(sp + (long)i * Dv);
      const float ki = ks[i], qi = qs[i];
      const float a = (KIND == GR_SSM) ? a_sc : as[i];
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
    out[((long)s * heads + h) * Dv + c] = acc + skip * vs[c];
  }
}

template <typename T, int KIND, int CPT>
void launch_gated_recurrence_cpt(float* out, const GRArgs<T>& A, float* state,
                                 const int* slots, const int* cu_q,
                                 const int* ctx_lens, int n_seqs, int chunk,
                                 int max_chunks, float* ws, float* wa,
                                 hipStream_t st) {
  const int D = A.D, Dv = A.Dv, heads = A.heads;
  const int Dd = (KIND == GR_SSM) ? 1 : D;
  constexpr int VS = GR_CG * CPT;
  const size_t lds = (size_t)(2 * GR_TC * D + GR_TC * (KIND == GR_SSM ? 2 : D)
                              + GR_TC * VS) * sizeof(float);
  const int vz = (Dv + VS - 1) / VS;
  if (ws == nullptr || max_chunks <= 1) {
    hipLaunchKernelGGL((gated_recurrence_kernel<T, KIND, CPT>),
                       dim3(n_seqs, heads, vz), dim3(256), lds, st, out, A,
                       state, slots, cu_q, ctx_lens, 0, 0, 1, nullptr, nullptr);
    return;
  }
  dim3 grid(n_seqs * max_chunks, heads, vz);
  hipLaunchKernelGGL((gated_recurrence_kernel<T, KIND, CPT>), grid, dim3(256),
                     lds, st, out, A, state, slots, cu_q, ctx_lens, 1, chunk,
                     max_chunks, ws, wa);
  const long per_seq = (long)heads * D * Dv;
  hipLaunchKernelGGL(gated_recurrence_scan_kernel,
                     dim3((unsigned)((per_seq + 255) / 256), n_seqs),
                     dim3(256), 0, st, ws, wa, state, slots, cu_q, ctx_lens,
                     heads, D, Dv, Dd, chunk, max_chunks);
  hipLaunchKernelGGL((gated_recurrence_kernel<T, KIND, CPT>), grid, dim3(256),
                     lds, st, out, A, state, slots, cu_q, ctx_lens, 2, chunk,
                     max_chunks, ws, wa);
}

template <typename T, int KIND>
void launch_gated_recurrence_kind(float* out, const GRArgs<T>& A, float* state,
                                  const int* slots, const int* cu_q,
                                  const int* ctx_lens, int n_seqs, int chunk,
                                  int max_chunks, float* ws, float* wa,
                                  hipStream_t st) {
  const int D = A.D, Dv = A.Dv, heads = A.heads;
  if (cu_q == nullptr && Dv % 4 == 0 && Dv <= 1024) {
    const int RG = 256 / (Dv / 4);
    const size_t l2 =
        (size_t)(3 * ((D + 3) & ~3) + Dv + RG * Dv) * sizeof(float);
    if (RG >= 1 && l2 <= 64 * 1024) {
      hipLaunchKernelGGL((gated_recurrence_decode_kernel<T, KIND>),
                         dim3(n_seqs, heads), dim3(256), l2, st, out, A, state,
                         slots, ctx_lens);
      return;
    }
  }
  // wide values and enough workgroups: four columns per thread (fewer LDS
  // reads per FMA). XLLM_RECURRENCE_COLS=1|4 fixes the choice (tuning knob).
  bool wide = Dv >= 48 &&
      (long)n_seqs * max_chunks * heads * ((Dv + 63) / 64) >= 512;
  if (const char* e = std::getenv("XLLM_RECURRENCE_COLS")) wide = e[0] == '4';
  if (wide)
    launch_gated_recurrence_cpt<T, KIND, 4>(out, A, state, slots, cu_q,
                                            ctx_lens, n_seqs, chunk,
                                            max_chunks, ws, wa, st);
  else
    launch_gated_recurrence_cpt<T, KIND, 1>(out, A, state, slots, cu_q,
                                            ctx_lens, n_seqs, chunk,
                                            max_chunks, ws, wa, st);
}

template <typename T>
void launch_gated_recurrence(int kind, float* out, const T* q, const T* k,
                             const T* v, const T* g, long q_stride,
                             long k_stride, long v_stride, long g_stride,
                             const float* p0, const float* p1, const float* p2,
                             float c0, float c1, float* state,
                             const int* slots, const int* cu_q,
                             const int* ctx_lens, int n_seqs, int heads,
                             int groups, int D, int Dv, int chunk,
                             int max_chunks, float* ws, float* wa,
                             hipStream_t st) {
  if (n_seqs == 0) return;
  GRArgs<T> A{q, k, v, g, q_stride, k_stride, v_stride, g_stride,
              p0, p1, p2, c0, c1, heads, groups, D, Dv};
  if (kind == GR_SSM)
    launch_gated_recurrence_kind<T, GR_SSM>(out, A, state, slots, cu_q,
                                            ctx_lens, n_seqs, chunk,
                                            max_chunks, ws, wa, st);
  else
    launch_gated_recurrence_kind<T, GR_GLA>(out, A, state, slots, cu_q,
                                            ctx_lens, n_seqs, chunk,
                                            max_chunks, ws, wa, st);
}

#define INST_GR(T)                                                            \
  template void launch_gated_recurrence<T>(                                   \
      int, float*, const T*, const T*, const T*, const T*, long, long, long,  \
      long, const float*, const float*, const float*, float, float, float*,   \
      const int*, const int*, const int*, int, int, int, int, int, int, int,  \
      float*, float*, hipStream_t);
INST_GR(float)
INST_GR(unsigned short)

}  // namespace hyb
}  // namespace xllm
