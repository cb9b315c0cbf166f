// Recurrences with per-sequence f32 state, advanced over the rows a step
// brings for each sequence (a prompt portion or one decoded token).
//
// A step brings, for sequence s, rows [loc[s], loc[s+1]) that continue it at
// position start = seq_len[s] - n.  State lives in slot-indexed f32 tensors;
// a sequence with start == 0 starts from zero state whatever its slot holds
// (slots are reused without clearing), slot < 0 marks a padding row of a
// captured decode bucket (zeros out, no state touched).
//
// matrix_scan<KIND>: state S [vdim, N] per (sequence, head), one column of
// the value axis per thread group:
//     S_t[j, :] = alpha_t * S_(t-1)[j, :] + beta_t * v_t[j] * k_t[:]
//     y_t[j]    = S_t[j, :] . q_t
//   KIND_SSD    alpha = exp(-exp(A_log) dt), beta = dt = softplus(raw + bias),
//               k = B, q = C (shared by the heads of a group), v = x,
//               y += D * x
//   KIND_MLSTM  log gates i, f (capped), running maximum m: alpha = exp(f + m
//               - m'), beta = exp(i - m'), a normaliser n_t = alpha n + beta k,
//               y = S q / (max(|n . q|, exp(-m')) + 1e-6)
//   KIND_HGRN2  a forget gate per state channel that also sets what is
//               written: S_t[j, i] = g_t[i] S_(t-1)[j, i] + (1 - g_t[i]) v_t[j],
//               g = l + (1 - l) sigmoid(f + b) with a lower bound l per
//               channel, y = S silu(q); a pointwise kernel ahead of the scan
//               writes g and silu(q) in f32 once per (row, head, channel)
// alpha, beta (and exp(-m')) are computed once per (row, head) by small gate
// kernels ahead of the scan (for the mLSTM a sequential pass over the rows
// carries the maximum), not by every thread of it.
// The N axis is split over NSP adjacent lanes, 16 state values per lane in
// registers (N <= 1024); a workgroup of 256 threads owns 256 / NSP value
// columns of one (sequence, head), or four times as many with four columns
// per thread (the key / query slices a thread loads then serve four columns).  State rows are stored [vdim, N] so that a
// wave loads and stores them as one contiguous run.  The value columns are
// independent of each other, so there is no barrier in the token loop: per
// token a thread does 32 FMAs per column and log2(NSP) DPP adds for its dot
// product.
//
// rglru_scan: elementwise linear recurrence, one thread per (sequence,
// channel), gates and decay computed in f32 on the fly.

#include "common.h"

#include <type_traits>

namespace {

constexpr int NPT = 16;   // state values per thread along N
enum { KIND_SSD = 0, KIND_MLSTM = 1, KIND_HGRN2 = 2 };

DEVINLINE float softplus_f(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }
DEVINLINE float logsigmoid_f(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }
DEVINLINE float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }

// Sum over NSP adjacent lanes (NSP a power of two, groups aligned), result in
// every lane.  Up to 16 lanes the partner values come through DPP modifiers on
// the adds (quad permutes, then the half-row and row mirrors — each mirror
// pairs a lane with one from the other, already uniform, half), which costs no
// LDS-crossbar round trip; wider groups finish with two shuffles.
template <int CTRL>
DEVINLINE float dpp_move(float v) {
  return __int_as_float(
      __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
template <int NSP>
DEVINLINE float lanes_sum(float x) {
  if (NSP >= 2) x += dpp_move<0xB1>(x);    // quad_perm [1,0,3,2]
  if (NSP >= 4) x += dpp_move<0x4E>(x);    // quad_perm [2,3,0,1]
  if (NSP >= 8) x += dpp_move<0x141>(x);   // row_half_mirror
  if (NSP >= 16) x += dpp_move<0x140>(x);  // row_mirror
  if (NSP >= 32) x += __shfl_xor(x, 16, WAVE_SIZE);
  if (NSP >= 64) x += __shfl_xor(x, 32, WAVE_SIZE);
  return x;
}

// 16 consecutive values p[n0 .. n0+16) of a row of length n_total as f32,
// zeros past the end
template <typename T>
DEVINLINE void load_slice(const T* __restrict__ p, int n0, int n_total, bool vec,
                          float* dst) {
  if (vec && n0 + NPT <= n_total) {
    constexpr int V = Vec16<T>::kElems;
#pragma unroll
    for (int i = 0; i < NPT; i += V) {
      const Vec16<T> v = load16(p + n0 + i);
#pragma unroll
      for (int u = 0; u < V; ++u) dst[i + u] = ScalarOps<T>::to_f32(v.data[u]);
    }
  } else {
#pragma unroll
    for (int i = 0; i < NPT; ++i)
      dst[i] = (n0 + i < n_total) ? ScalarOps<T>::to_f32(p[n0 + i]) : 0.f;
  }
}

struct ScanArgs {
  // rows
  const void* q; const void* k; const void* v;
  long q_st, k_st, v_st;             // row strides (elements)
  const void* g0; const void* g1;    // SSD: raw dt; mLSTM: i_pre, f_pre  [T, H] strided
  long g0_st, g1_st;
  const float* p0; const float* p1; const float* p2;  // SSD: dt_bias, A_log, D; mLSTM: i_bias, f_bias
  float cap, q_scale;
  float4* gates; int rows;           // per (row, head): alpha, beta, exp(-m), -  (f32)
  float* y; long y_st;               // [T, H*vdim] f32
  float* s_state; float* n_state; float* m_state;
  const int* loc; const int* seq_lens; const int* slots;
  int heads, vdim, nk, per_group;    // nk = N (SSD) or dim (mLSTM); heads per k/q group
  int vec_ok;
};

// Gates per (row, head), computed once instead of by every thread of the scan.
// Pointwise part: SSD alpha = exp(-exp(A_log) dt), beta = dt; mLSTM the capped
// log gates (i in .x, f in .y) that the sequential pass below turns into
// alpha, beta and exp(-m).
template <typename T, int KIND>
__global__ void scan_gates_pointwise_kernel(ScanArgs a) {
  const long idx = blockIdx.x * (long)blockDim.x + threadIdx.x;
  if (idx >= (long)a.rows * a.heads) return;
  const long row = idx / a.heads;
  const int h = (int)(idx - row * a.heads);
  const float g0 = ScalarOps<T>::to_f32(reinterpret_cast<const T*>(a.g0)[row * a.g0_st + h]);
  float4 out = make_float4(0.f, 0.f, 1.f, 0.f);
  if (KIND == KIND_SSD) {
    const float dt = softplus_f(g0 + a.p0[h]);
    out.x = expf(-expf(a.p1[h]) * dt);
    out.y = dt;
  } else {
    const float g1 = ScalarOps<T>::to_f32(reinterpret_cast<const T*>(a.g1)[row * a.g1_st + h]);
    out.x = a.cap * tanhf((g0 + a.p0[h]) / a.cap);
    out.y = logsigmoid_f(a.cap * tanhf((g1 + a.p1[h]) / a.cap));
  }
  a.gates[idx] = out;
}

// mLSTM: one thread per (sequence, head) walks the step's rows with the
// running maximum (0 at position 0): m' = max(f + m, i), alpha = exp(f + m -
// m'), beta = exp(i - m'), and stores exp(-m') for the output's denominator.
// Leaves the new maximum in m_state; nothing else reads m_state in the step.
__global__ void mlstm_gates_scan_kernel(ScanArgs a, int nseq) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= nseq * a.heads) return;
  const int s = idx / a.heads;
  const int h = idx - s * a.heads;
  const int row0 = a.loc[s];
  const int n = a.loc[s + 1] - row0;
  const int slot = a.slots[s];
  if (n <= 0 || slot < 0) return;
  float* mp = a.m_state + (long)slot * a.heads + h;
  float m = (a.seq_lens[s] - n) > 0 ? *mp : 0.f;
  for (int r = 0; r < n; ++r) {
    float4* g = a.gates + (long)(row0 + r) * a.heads + h;
    const float ig = g->x, fg = g->y;
    const float m_new = fmaxf(fg + m, ig);
    *g = make_float4(expf(fg + m - m_new), expf(ig - m_new), expf(-m_new), 0.f);
    m = m_new;
  }
  *mp = m;
}

template <typename T, int KIND, int NSP, int VPT>
__global__ __launch_bounds__(256) void matrix_scan_kernel(ScanArgs a) {
  constexpr int JW = 256 / NSP;            // thread groups per workgroup
  const int s = blockIdx.x / a.heads;
  const int h = blockIdx.x % a.heads;
  const int ns = threadIdx.x % NSP;
  const int jbase = (blockIdx.y * JW + threadIdx.x / NSP) * VPT;   // first value column
  const int row0 = a.loc[s];
  const int n = a.loc[s + 1] - row0;
  if (n <= 0) return;
  const int slot = a.slots[s];
  if (slot < 0) {
    if (ns == 0)
      for (int r = 0; r < n; ++r)
#pragma unroll
        for (int c = 0; c < VPT; ++c)
          if (jbase + c < a.vdim)
            a.y[(long)(row0 + r) * a.y_st + (long)h * a.vdim + jbase + c] = 0.f;
    return;
  }
  const int start = a.seq_lens[s] - n;
  const int n0 = ns * NPT;
  const int grp = h / a.per_group;
  const bool vec = a.vec_ok != 0;

  // columns past vdim are clamped: they compute and never store
  int jc[VPT];
#pragma unroll
  for (int c = 0; c < VPT; ++c) jc[c] = min(jbase + c, a.vdim - 1);

  float S[VPT][NPT], nst[NPT];
  float* sbase = a.s_state + ((long)slot * a.heads + h) * a.vdim * a.nk;
  const float* nrow = KIND == KIND_MLSTM ? a.n_state + ((long)slot * a.heads + h) * a.nk : nullptr;
  if (start > 0) {
#pragma unroll
    for (int c = 0; c < VPT; ++c) load_slice<float>(sbase + (long)jc[c] * a.nk, n0, a.nk, vec, S[c]);
    if (KIND == KIND_MLSTM) load_slice<float>(nrow, n0, a.nk, vec, nst);
  } else {
#pragma unroll
    for (int i = 0; i < NPT; ++i) {
      nst[i] = 0.f;
#pragma unroll
      for (int c = 0; c < VPT; ++c) S[c][i] = 0.f;
    }
  }

  const float c2 = KIND == KIND_SSD ? a.p2[h] : 0.f;   // D
  const float4* gp = a.gates + h;
  // HGRN2 reads its gate and activated query from the f32 rows of the pre-pass
  using KQ = typename std::conditional<KIND == KIND_HGRN2, float, T>::type;
  const KQ* qp = reinterpret_cast<const KQ*>(a.q) + (long)grp * a.nk;
  const KQ* kp = reinterpret_cast<const KQ*>(a.k) + (long)grp * a.nk;
  const T* vp = reinterpret_cast<const T*>(a.v) + (long)h * a.vdim;

  // the next row's inputs are loaded while this row is computed: with two
  // waves per SIMD the load latency is otherwise paid once per token
  float kk[NPT], qq[NPT], vj[VPT];
  float4 gt;
  auto load_row = [&](long row, float* k_, float* q_, float* v_, float4& g_) {
    load_slice<KQ>(kp + row * a.k_st, n0, a.nk, vec, k_);
    load_slice<KQ>(qp + row * a.q_st, n0, a.nk, vec, q_);
#pragma unroll
    for (int c = 0; c < VPT; ++c) v_[c] = ScalarOps<T>::to_f32(vp[row * a.v_st + jc[c]]);
    g_ = KIND == KIND_HGRN2 ? make_float4(0.f, 0.f, 0.f, 0.f) : gp[row * a.heads];
  };
  load_row(row0, kk, qq, vj, gt);
  for (int r = 0; r < n; ++r) {
    const long row = row0 + r;
    float kn[NPT], qn[NPT], vn[VPT];
    float4 gn;
    const bool more = r + 1 < n;       // uniform over the workgroup
    if (more) load_row(row + 1, kn, qn, vn, gn);
    const float alpha = gt.x, beta = gt.y;
    float dot[VPT], ndot = 0.f;
#pragma unroll
    for (int c = 0; c < VPT; ++c) dot[c] = 0.f;
#pragma unroll
    for (int i = 0; i < NPT; ++i) {
      const float al = KIND == KIND_HGRN2 ? kk[i] : alpha;
      const float bk = KIND == KIND_HGRN2 ? 1.0f - kk[i] : beta * kk[i];
      if (KIND == KIND_MLSTM) {
        nst[i] = alpha * nst[i] + bk;
        ndot += nst[i] * qq[i];
      }
#pragma unroll
      for (int c = 0; c < VPT; ++c) {
        S[c][i] = al * S[c][i] + bk * vj[c];
        dot[c] += S[c][i] * qq[i];
      }
    }
    float den = 1.f;    // mLSTM: the query scale is applied to the two sums
    if (KIND == KIND_MLSTM) {
      ndot = lanes_sum<NSP>(ndot) * a.q_scale;
      den = a.q_scale / (fmaxf(fabsf(ndot), gt.z) + 1e-6f);
    }
#pragma unroll
    for (int c = 0; c < VPT; ++c) {
      const float d = lanes_sum<NSP>(dot[c]);
      const float yv = KIND == KIND_MLSTM ? d * den : d + c2 * vj[c];
      if (ns == 0 && jbase + c < a.vdim)
        a.y[row * a.y_st + (long)h * a.vdim + jbase + c] = yv;
    }
    if (more) {
#pragma unroll
      for (int i = 0; i < NPT; ++i) { kk[i] = kn[i]; qq[i] = qn[i]; }
#pragma unroll
      for (int c = 0; c < VPT; ++c) vj[c] = vn[c];
      gt = gn;
    }
  }

#pragma unroll
  for (int c = 0; c < VPT; ++c) {
    if (jbase + c >= a.vdim) continue;
    float* srow = sbase + (long)(jbase + c) * a.nk;
    if (vec && n0 + NPT <= a.nk) {
#pragma unroll
      for (int i = 0; i < NPT; i += 4)
        *reinterpret_cast<float4*>(srow + n0 + i) =
            make_float4(S[c][i], S[c][i + 1], S[c][i + 2], S[c][i + 3]);
    } else {
#pragma unroll
      for (int i = 0; i < NPT; ++i)
        if (n0 + i < a.nk) srow[n0 + i] = S[c][i];
    }
  }
  // the normaliser n is read by every workgroup of this (sequence, head) and
  // therefore advanced by a kernel of its own, after this one, on the same
  // stream
}

// Advances the mLSTM normaliser n [slots, H, dim] over the step's rows with the
// precomputed gates: one workgroup per (sequence, head), one thread per key dim.
template <typename T>
__global__ __launch_bounds__(256) void mlstm_norm_state_kernel(ScanArgs a) {
  const int s = blockIdx.x / a.heads;
  const int h = blockIdx.x % a.heads;
  const int row0 = a.loc[s];
  const int n = a.loc[s + 1] - row0;
  const int slot = a.slots[s];
  if (n <= 0 || slot < 0) return;
  const int start = a.seq_lens[s] - n;
  const T* kp = reinterpret_cast<const T*>(a.k) + (long)h * a.nk;
  const float4* gp = a.gates + h;
  float* nrow = a.n_state + ((long)slot * a.heads + h) * a.nk;
  for (int d = threadIdx.x; d < a.nk; d += blockDim.x) {
    float nv = start > 0 ? nrow[d] : 0.f;
    for (int r = 0; r < n; ++r) {
      const long row = row0 + r;
      const float4 gt = gp[row * a.heads];
      nv = gt.x * nv + gt.y * ScalarOps<T>::to_f32(kp[row * a.k_st + d]);
    }
    nrow[d] = nv;
  }
}

// HGRN2 pre-pass: gq [T, 2, H * dim] f32 = (l + (1 - l) sigmoid(f + b), silu(q))
template <typename T>
__global__ __launch_bounds__(256) void hgrn2_gates_kernel(
    float* __restrict__ gq, const T* __restrict__ q, long q_st,
    const T* __restrict__ f, long f_st, const float* __restrict__ f_bias,
    const float* __restrict__ lower, long rows, int hd) {
  const long idx = blockIdx.x * (long)blockDim.x + threadIdx.x;
  if (idx >= rows * hd) return;
  const long row = idx / hd;
  const int c = (int)(idx - row * hd);
  const float lo = lower[c];
  const float fv = ScalarOps<T>::to_f32(f[row * f_st + c]) + f_bias[c];
  const float qv = ScalarOps<T>::to_f32(q[row * q_st + c]);
  gq[row * 2 * hd + c] = lo + (1.0f - lo) * sigmoid_f(fv);
  gq[row * 2 * hd + hd + c] = qv * sigmoid_f(qv);
}

template <typename T, int KIND>
void launch_matrix_scan(const ScanArgs& a, int nseq, hipStream_t stream) {
  const int nslices = (a.nk + NPT - 1) / NPT;
  int nsp = 1;
  while (nsp < nslices) nsp <<= 1;
  // four (or two) value columns per thread when that still fills a workgroup: the key
  // and query slices a thread loads then serve four state columns
#define SCAN_CASE(P)                                                           \
  case P: {                                                                    \
    constexpr int JW = 256 / P;                                                \
    if (a.vdim >= 4 * JW) {                                                    \
      dim3 grid(nseq * a.heads, (a.vdim + 4 * JW - 1) / (4 * JW));             \
      matrix_scan_kernel<T, KIND, P, 4><<<grid, 256, 0, stream>>>(a);          \
    } else if (a.vdim >= 2 * JW) {                                             \
      dim3 grid(nseq * a.heads, (a.vdim + 2 * JW - 1) / (2 * JW));             \
      matrix_scan_kernel<T, KIND, P, 2><<<grid, 256, 0, stream>>>(a);          \
    } else {                                                                   \
      dim3 grid(nseq * a.heads, (a.vdim + JW - 1) / JW);                       \
      matrix_scan_kernel<T, KIND, P, 1><<<grid, 256, 0, stream>>>(a);          \
    }                                                                          \
    break;                                                                     \
  }
  switch (nsp) {
    SCAN_CASE(1) SCAN_CASE(2) SCAN_CASE(4) SCAN_CASE(8) SCAN_CASE(16)
    SCAN_CASE(32) SCAN_CASE(64)
    default: break;   // the binding refuses N > 1024
  }
#undef SCAN_CASE
}

template <typename T>
__global__ __launch_bounds__(256) void rglru_scan_kernel(
    T* __restrict__ out, const T* __restrict__ u, const T* __restrict__ r_pre,
    const T* __restrict__ i_pre, const float* __restrict__ r_bias,
    const float* __restrict__ i_bias, const float* __restrict__ lam, float gate_c,
    const T* __restrict__ y_branch, float* __restrict__ state,
    const int* __restrict__ loc, const int* __restrict__ seq_lens,
    const int* __restrict__ slots, int width) {
  const int s = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= width) return;
  const int row0 = loc[s];
  const int n = loc[s + 1] - row0;
  if (n <= 0) return;
  const int slot = slots[s];
  if (slot < 0) {
    for (int r = 0; r < n; ++r) out[(long)(row0 + r) * width + c] = ScalarOps<T>::from_f32(0.f);
    return;
  }
  const int start = seq_lens[s] - n;
  float S = start > 0 ? state[(long)slot * width + c] : 0.f;
  const float rb = r_bias[c], ib = i_bias[c];
  const float sp = -gate_c * softplus_f(lam[c]);
  for (int r = 0; r < n; ++r) {
    const long o = (long)(row0 + r) * width + c;
    const float uv = ScalarOps<T>::to_f32(u[o]);
    const float rg = sigmoid_f(ScalarOps<T>::to_f32(r_pre[o]) + rb);
    const float ig = sigmoid_f(ScalarOps<T>::to_f32(i_pre[o]) + ib);
    const float av = expf(sp * rg);
    S = av * S + sqrtf(1.0f - av * av) * ig * uv;
    out[o] = ScalarOps<T>::from_f32(S * ScalarOps<T>::to_f32(y_branch[o]));
  }
  state[(long)slot * width + c] = S;
}

}  // namespace

template <typename T>
void launch_ssd_scan(float* y, const T* xbc, long xbc_st, const T* dt, long dt_st,
                     const float* dt_bias, const float* a_log, const float* d_skip,
                     float* state, const int* loc, const int* seq_lens,
                     const int* slots, int nseq, int heads, int vdim, int nstate,
                     int groups, int vec_ok, float* gates, int rows,
                     hipStream_t stream) {
  const int inner = heads * vdim;
  ScanArgs a{};
  a.gates = reinterpret_cast<float4*>(gates); a.rows = rows;
  a.v = xbc;                                  a.v_st = xbc_st;
  a.k = xbc + inner;                          a.k_st = xbc_st;
  a.q = xbc + inner + (long)groups * nstate;  a.q_st = xbc_st;
  a.g0 = dt; a.g0_st = dt_st;
  a.p0 = dt_bias; a.p1 = a_log; a.p2 = d_skip;
  a.y = y; a.y_st = inner;
  a.s_state = state;
  a.loc = loc; a.seq_lens = seq_lens; a.slots = slots;
  a.heads = heads; a.vdim = vdim; a.nk = nstate; a.per_group = heads / groups;
  a.vec_ok = vec_ok;
  const long ng = (long)rows * heads;
  scan_gates_pointwise_kernel<T, KIND_SSD><<<(int)((ng + 255) / 256), 256, 0, stream>>>(a);
  launch_matrix_scan<T, KIND_SSD>(a, nseq, stream);
}

template <typename T>
void launch_mlstm_scan(float* o, const T* q, long q_st, const T* k, long k_st,
                       const T* v, long v_st, const T* i_pre, long i_st,
                       const T* f_pre, long f_st, const float* i_bias,
                       const float* f_bias, float cap, float q_scale,
                       float* s_state, float* n_state, float* m_state,
                       const int* loc, const int* seq_lens, const int* slots,
                       int nseq, int heads, int dim, int vdim, int vec_ok,
                       float* gates, int rows, hipStream_t stream) {
  ScanArgs a{};
  a.gates = reinterpret_cast<float4*>(gates); a.rows = rows;
  a.q = q; a.q_st = q_st; a.k = k; a.k_st = k_st; a.v = v; a.v_st = v_st;
  a.g0 = i_pre; a.g0_st = i_st; a.g1 = f_pre; a.g1_st = f_st;
  a.p0 = i_bias; a.p1 = f_bias;
  a.cap = cap; a.q_scale = q_scale;
  a.y = o; a.y_st = (long)heads * vdim;
  a.s_state = s_state; a.n_state = n_state; a.m_state = m_state;
  a.loc = loc; a.seq_lens = seq_lens; a.slots = slots;
  a.heads = heads; a.vdim = vdim; a.nk = dim; a.per_group = 1;
  a.vec_ok = vec_ok;
  const long ng = (long)rows * heads;
  scan_gates_pointwise_kernel<T, KIND_MLSTM><<<(int)((ng + 255) / 256), 256, 0, stream>>>(a);
  mlstm_gates_scan_kernel<<<(nseq * heads + 63) / 64, 64, 0, stream>>>(a, nseq);
  launch_matrix_scan<T, KIND_MLSTM>(a, nseq, stream);
  const int block = dim >= 256 ? 256 : ((dim + 63) / 64) * 64;
  mlstm_norm_state_kernel<T><<<nseq * heads, block, 0, stream>>>(a);
}

template <typename T>
void launch_hgrn2_scan(float* o, const T* q, long q_st, const T* f, long f_st,
                       const T* v, long v_st, const float* f_bias,
                       const float* lower, float* state, const int* loc,
                       const int* seq_lens, const int* slots, int nseq, int heads,
                       int dim, int vdim, int vec_ok, float* gq, int rows,
                       hipStream_t stream) {
  const int hd = heads * dim;
  const long total = (long)rows * hd;
  hgrn2_gates_kernel<T><<<(int)((total + 255) / 256), 256, 0, stream>>>(
      gq, q, q_st, f, f_st, f_bias, lower, rows, hd);
  ScanArgs a{};
  a.rows = rows;
  a.k = gq;      a.k_st = 2L * hd;
  a.q = gq + hd; a.q_st = 2L * hd;
  a.v = v;       a.v_st = v_st;
  a.y = o; a.y_st = (long)heads * vdim;
  a.s_state = state;
  a.loc = loc; a.seq_lens = seq_lens; a.slots = slots;
  a.heads = heads; a.vdim = vdim; a.nk = dim; a.per_group = 1;
  a.vec_ok = vec_ok;
  launch_matrix_scan<T, KIND_HGRN2>(a, nseq, stream);
}

template <typename T>
void launch_rglru_scan(T* out, const T* u, const T* r_pre, const T* i_pre,
                       const float* r_bias, const float* i_bias, const float* lam,
                       float gate_c, const T* y_branch, float* state,
                       const int* loc, const int* seq_lens, const int* slots,
                       int nseq, int width, hipStream_t stream) {
  const int block = width >= 256 ? 256 : ((width + 63) / 64) * 64;
  dim3 grid(nseq, (width + block - 1) / block);
  rglru_scan_kernel<T><<<grid, block, 0, stream>>>(
      out, u, r_pre, i_pre, r_bias, i_bias, lam, gate_c, y_branch, state, loc,
      seq_lens, slots, width);
}

#define INSTANTIATE(T)                                                          \
  template void launch_ssd_scan<T>(float*, const T*, long, const T*, long,      \
                                   const float*, const float*, const float*,    \
                                   float*, const int*, const int*, const int*,  \
                                   int, int, int, int, int, int, float*, int,   \
                                   hipStream_t);                                \
  template void launch_mlstm_scan<T>(                                           \
      float*, const T*, long, const T*, long, const T*, long, const T*, long,   \
      const T*, long, const float*, const float*, float, float, float*, float*, \
      float*, const int*, const int*, const int*, int, int, int, int, int,      \
      float*, int, hipStream_t);                                                \
  template void launch_hgrn2_scan<T>(float*, const T*, long, const T*, long,    \
                                     const T*, long, const float*, const float*,\
                                     float*, const int*, const int*, const int*,\
                                     int, int, int, int, int, float*, int,      \
                                     hipStream_t);                              \
  template void launch_rglru_scan<T>(T*, const T*, const T*, const T*,          \
                                     const float*, const float*, const float*,  \
                                     float, const T*, float*, const int*,       \
                                     const int*, const int*, int, int,          \
                                     hipStream_t);
INSTANTIATE(float)
INSTANTIATE(__hip_bfloat16)
