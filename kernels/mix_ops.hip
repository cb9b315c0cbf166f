// Row kernels around the mixers of a model whose sublayers read the f32
// residual stream itself: token shift with a carried row per sequence,
// query/key norm + half-split rotation + paged cache write, the combination
// of the two maps of differential attention, RMS norm in equal groups, and
// the gated activation of experts whose input carries the routing weight.
// Statistics, angles, gates and sums are f32 whatever the storage type.

#include "common.h"

namespace {

DEVINLINE float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }

// ---------------------------------------------------------------------------
// token shift:  out_t = x_t + (x_(t-1) - x_t) * w
// One workgroup per row.  The row before a portion's first row is the
// sequence's carried row (zero at position 0); the workgroup of that first row
// also stores the portion's last row as the new carried row, so the carried
// row is read and written by the same threads.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void token_shift_state_kernel(
    T* __restrict__ out, const float* __restrict__ x, const float* __restrict__ w,
    float* __restrict__ state, const int* __restrict__ loc,
    const int* __restrict__ seq_lens, const int* __restrict__ slots, int nseq,
    int width) {
  const int row = blockIdx.x;
  int lo = 0, hi = nseq;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (loc[mid] <= row) lo = mid; else hi = mid;
  }
  // the last sequence that starts at or before this row is the one that has it
  // (sequences without rows share their start with the next one)
  const int s = lo;
  const int row0 = loc[s];
  const int n = loc[s + 1] - row0;
  const int slot = slots[s];
  T* orow = out + (long)row * width;
  if (slot < 0 || row >= row0 + n) {
    for (int c = threadIdx.x; c < width; c += blockDim.x) orow[c] = ScalarOps<T>::from_f32(0.f);
    return;
  }
  const float* xr = x + (long)row * width;
  const bool first = row == row0;
  const bool from_state = first && (seq_lens[s] - n) > 0;
  float* st = state + (long)slot * width;
  const float* prev = first ? st : xr - width;
  const float* last = x + (long)(row0 + n - 1) * width;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float xv = xr[c];
    const float pv = (first && !from_state) ? 0.f : prev[c];
    orow[c] = ScalarOps<T>::from_f32(xv + (pv - xv) * w[c]);
    if (first) st[c] = last[c];
  }
}

// ---------------------------------------------------------------------------
// query/key RMS norm per head (one weight for all heads), rotation of the
// first rot dims (dim i with i + rot/2), keys and values into the paged cache.
// One workgroup per token, one wave per head at a time; the normed head sits
// in LDS so that a lane finds the partner of its dim.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void qk_norm_rope_cache_write_kernel(
    T* __restrict__ q_out, const T* __restrict__ q, long q_st,
    const T* __restrict__ k, long k_st, const T* __restrict__ v, long v_st,
    const float* __restrict__ qw, const float* __restrict__ kw, float eps,
    const long* __restrict__ positions, const float* __restrict__ inv_freq,
    int rot, T* __restrict__ k_cache, T* __restrict__ v_cache,
    const long* __restrict__ slot_mapping, int heads, int kv_heads, int v_heads,
    int dim, int vdim) {
  extern __shared__ float smem[];
  const int tok = blockIdx.x;
  const int lane = threadIdx.x & (WAVE_SIZE - 1);
  const int wave = threadIdx.x / WAVE_SIZE;
  const int nwaves = blockDim.x / WAVE_SIZE;
  float* buf = smem + wave * dim;
  const float pos = (float)positions[tok];
  const long slot = slot_mapping[tok];
  const int half = rot / 2;
  for (int hb = 0; hb < heads + kv_heads; hb += nwaves) {
    // the last round may leave waves without a head: they redo the last one
    const int hh = min(hb + wave, heads + kv_heads - 1);
    const bool is_q = hh < heads;
    const T* src = is_q ? q + tok * q_st + (long)hh * dim
                        : k + tok * k_st + (long)(hh - heads) * dim;
    const float* wt = is_q ? qw : kw;
    float ss = 0.f;
    for (int c = lane; c < dim; c += WAVE_SIZE) {
      const float f = ScalarOps<T>::to_f32(src[c]);
      buf[c] = f;
      ss += f * f;
    }
    ss = wave_reduce_sum(ss);
    const float inv = rsqrtf(ss / (float)dim + eps);
    for (int c = lane; c < dim; c += WAVE_SIZE) buf[c] = buf[c] * inv * wt[c];
    __syncthreads();
    T* dst = nullptr;
    if (is_q) dst = q_out + ((long)tok * heads + hh) * dim;
    else if (slot >= 0) dst = k_cache + (slot * kv_heads + (hh - heads)) * dim;
    if (dst != nullptr) {
      for (int c = lane; c < dim; c += WAVE_SIZE) {
        float val = buf[c];
        if (c < rot) {
          const int i = c < half ? c : c - half;
          float sn, cs;
          sincosf(pos * inv_freq[i], &sn, &cs);
          const float a = buf[i], b = buf[i + half];
          val = c < half ? a * cs - b * sn : b * cs + a * sn;
        }
        dst[c] = ScalarOps<T>::from_f32(val);
      }
    }
    __syncthreads();
  }
  if (slot >= 0) {
    const T* vr = v + tok * v_st;
    T* vd = v_cache + slot * (long)v_heads * vdim;
    for (int c = threadIdx.x; c < v_heads * vdim; c += blockDim.x) vd[c] = vr[c];
  }
}

// ---------------------------------------------------------------------------
// differential combination: a [T, 2, H, vdim] f32 ->
// (a0 - lam a1) / rms * out_scale * sigmoid(gate[t, h])   [T, H * vdim]
// One wave per (token, head).
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void diff_combine_kernel(
    T* __restrict__ out, const float* __restrict__ a, float lam, float out_scale,
    float eps, const T* __restrict__ gate, long g_st, int tokens, int heads,
    int vdim) {
  const int lane = threadIdx.x & (WAVE_SIZE - 1);
  const long idx = blockIdx.x * (long)(blockDim.x / WAVE_SIZE) + threadIdx.x / WAVE_SIZE;
  if (idx >= (long)tokens * heads) return;
  const long t = idx / heads;
  const int h = (int)(idx - t * heads);
  const float* a0 = a + ((t * 2) * heads + h) * vdim;
  const float* a1 = a + ((t * 2 + 1) * heads + h) * vdim;
  float ss = 0.f;
  for (int c = lane; c < vdim; c += WAVE_SIZE) {
    const float o = a0[c] - lam * a1[c];
    ss += o * o;
  }
  ss = wave_reduce_sum(ss);
  float mul = rsqrtf(ss / (float)vdim + eps) * out_scale;
  if (gate != nullptr) mul *= sigmoid_f(ScalarOps<T>::to_f32(gate[t * g_st + h]));
  T* orow = out + (t * heads + h) * vdim;
  for (int c = lane; c < vdim; c += WAVE_SIZE)
    orow[c] = ScalarOps<T>::from_f32((a0[c] - lam * a1[c]) * mul);
}

// ---------------------------------------------------------------------------
// RMS norm of f32 rows in equal groups, times a weight per channel.
// One wave per (row, group).
// ---------------------------------------------------------------------------
template <typename T, typename I>
__global__ __launch_bounds__(256) void group_rms_norm_kernel(
    T* __restrict__ out, const I* __restrict__ y, const float* __restrict__ w,
    float eps, long rows, int groups, int gsize) {
  const int lane = threadIdx.x & (WAVE_SIZE - 1);
  const long idx = blockIdx.x * (long)(blockDim.x / WAVE_SIZE) + threadIdx.x / WAVE_SIZE;
  if (idx >= rows * groups) return;
  const int g = (int)(idx % groups);
  const I* yr = y + idx * gsize;
  const float* wr = w + (long)g * gsize;
  float ss = 0.f;
  for (int c = lane; c < gsize; c += WAVE_SIZE) {
    const float f = ScalarOps<I>::to_f32(yr[c]);
    ss += f * f;
  }
  ss = wave_reduce_sum(ss);
  const float inv = rsqrtf(ss / (float)gsize + eps);
  T* orow = out + idx * gsize;
  for (int c = lane; c < gsize; c += WAVE_SIZE)
    orow[c] = ScalarOps<T>::from_f32(ScalarOps<I>::to_f32(yr[c]) * inv * wr[c]);
}

// ---------------------------------------------------------------------------
// gu [T, E, 2, ff] -> out [T, E, ff] = silu(w g) * (w u), w = scale[t, e] f32
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void silu_mul_scaled_kernel(
    T* __restrict__ out, const T* __restrict__ gu, const float* __restrict__ scale,
    long total, int experts, int ff) {
  const long idx = blockIdx.x * (long)blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const long te = idx / ff;             // t * experts + e
  const int j = (int)(idx - te * ff);
  const float w = scale[te];
  float r = 0.f;
  if (w != 0.f) {
    const T* p = gu + te * 2 * ff;
    const float g = w * ScalarOps<T>::to_f32(p[j]);
    const float u = w * ScalarOps<T>::to_f32(p[ff + j]);
    r = g * sigmoid_f(g) * u;
  }
  out[idx] = ScalarOps<T>::from_f32(r);
}

}  // namespace

template <typename T>
void launch_token_shift_state(T* out, const float* x, const float* w, float* state,
                              const int* loc, const int* seq_lens, const int* slots,
                              int nseq, int rows, int width, hipStream_t s) {
  const int block = width >= 256 ? 256 : ((width + 63) / 64) * 64;
  token_shift_state_kernel<T><<<rows, block, 0, s>>>(out, x, w, state, loc, seq_lens,
                                                    slots, nseq, width);
}

template <typename T>
void launch_qk_norm_rope_cache_write(T* q_out, const T* q, long q_st, const T* k,
                                     long k_st, const T* v, long v_st,
                                     const float* qw, const float* kw, float eps,
                                     const long* positions, const float* inv_freq,
                                     int rot, T* k_cache, T* v_cache,
                                     const long* slot_mapping, int tokens, int heads,
                                     int kv_heads, int v_heads, int dim, int vdim,
                                     hipStream_t s) {
  const int waves = 4;
  qk_norm_rope_cache_write_kernel<T>
      <<<tokens, waves * WAVE_SIZE, sizeof(float) * waves * dim, s>>>(
          q_out, q, q_st, k, k_st, v, v_st, qw, kw, eps, positions, inv_freq, rot,
          k_cache, v_cache, slot_mapping, heads, kv_heads, v_heads, dim, vdim);
}

template <typename T>
void launch_diff_combine(T* out, const float* a, float lam, float out_scale,
                         float eps, const T* gate, long g_st, int tokens, int heads,
                         int vdim, hipStream_t s) {
  const long n = (long)tokens * heads;
  diff_combine_kernel<T><<<(int)((n + 3) / 4), 256, 0, s>>>(
      out, a, lam, out_scale, eps, gate, g_st, tokens, heads, vdim);
}

template <typename T, typename I>
void launch_group_rms_norm(T* out, const I* y, const float* w, float eps, long rows,
                           int groups, int gsize, hipStream_t s) {
  const long n = rows * groups;
  group_rms_norm_kernel<T, I><<<(int)((n + 3) / 4), 256, 0, s>>>(out, y, w, eps, rows,
                                                               groups, gsize);
}

template <typename T>
void launch_silu_mul_scaled(T* out, const T* gu, const float* scale, long tokens,
                            int experts, int ff, hipStream_t s) {
  const long total = tokens * experts * ff;
  silu_mul_scaled_kernel<T><<<(int)((total + 255) / 256), 256, 0, s>>>(
      out, gu, scale, total, experts, ff);
}

#define INSTANTIATE(T)                                                            \
  template void launch_token_shift_state<T>(T*, const float*, const float*, float*, \
                                            const int*, const int*, const int*,   \
                                            int, int, int, hipStream_t);          \
  template void launch_qk_norm_rope_cache_write<T>(                               \
      T*, const T*, long, const T*, long, const T*, long, const float*,           \
      const float*, float, const long*, const float*, int, T*, T*, const long*,   \
      int, int, int, int, int, int, hipStream_t);                                 \
  template void launch_diff_combine<T>(T*, const float*, float, float, float,     \
                                       const T*, long, int, int, int,             \
                                       hipStream_t);                              \
  template void launch_group_rms_norm<T, float>(T*, const float*, const float*,   \
                                                float, long, int, int,            \
                                                hipStream_t);                     \
  template void launch_silu_mul_scaled<T>(T*, const T*, const float*, long, int,  \
                                          int, hipStream_t);
INSTANTIATE(float)
INSTANTIATE(__hip_bfloat16)
template void launch_group_rms_norm<__hip_bfloat16, __hip_bfloat16>(
    __hip_bfloat16*, const __hip_bfloat16*, const float*, float, long, int, int,
    hipStream_t);
