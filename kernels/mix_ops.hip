// Row kernels around the mixers of a model whose sublayers read the f32
// residual stream itself: token shift with a carried row per sequence,
// query/key norm + half-split rotation + paged cache write, the combination
// of the two maps of differential attention, RMS norm in equal groups, and
// the gated activation of experts whose input carries the routing weight.
// Statistics, angles, gates and sums are f32 whatever the storage type.

#include "common.h"

namespace {

DEVINLINE float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }

// four consecutive elements as f32 (16-byte f32 or 8-byte bf16 accesses)
struct F4 { float v[4]; };
template <typename T> struct Pack4;
template <> struct Pack4<float> {
  static DEVINLINE F4 load(const float* p) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    return F4{{t.x, t.y, t.z, t.w}};
  }
  static DEVINLINE void store(float* p, const F4& f) {
    *reinterpret_cast<float4*>(p) = make_float4(f.v[0], f.v[1], f.v[2], f.v[3]);
  }
};
template <> struct Pack4<__hip_bfloat16> {
  static DEVINLINE F4 load(const __hip_bfloat16* p) {
    const uint2 t = *reinterpret_cast<const uint2*>(p);
    F4 f;
    f.v[0] = __uint_as_float(t.x << 16);
    f.v[1] = __uint_as_float(t.x & 0xffff0000u);
    f.v[2] = __uint_as_float(t.y << 16);
    f.v[3] = __uint_as_float(t.y & 0xffff0000u);
    return f;
  }
  static DEVINLINE void store(__hip_bfloat16* p, const F4& f) {
    union { __hip_bfloat16 h[4]; uint2 u; } o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o.h[i] = __float2bfloat16(f.v[i]);
    *reinterpret_cast<uint2*>(p) = o.u;
  }
};

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
    int width, int vec) {
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
  const bool zero_prev = first && !from_state;
  if (vec) {   // width % 4 == 0, 16-byte aligned rows
    for (int c = threadIdx.x * 4; c < width; c += blockDim.x * 4) {
      const F4 xv = Pack4<float>::load(xr + c);
      F4 pv = xv;
      if (zero_prev) pv = F4{{0.f, 0.f, 0.f, 0.f}};
      else pv = Pack4<float>::load(prev + c);
      const F4 wv = Pack4<float>::load(w + c);
      F4 o;
#pragma unroll
      for (int k = 0; k < 4; ++k) o.v[k] = xv.v[k] + (pv.v[k] - xv.v[k]) * wv.v[k];
      Pack4<T>::store(orow + c, o);
      if (first) Pack4<float>::store(st + c, Pack4<float>::load(last + c));
    }
    return;
  }
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float xv = xr[c];
    const float pv = zero_prev ? 0.f : prev[c];
    orow[c] = ScalarOps<T>::from_f32(xv + (pv - xv) * w[c]);
    if (first) st[c] = last[c];
  }
}

// ---------------------------------------------------------------------------
// query/key RMS norm per head (one weight for all heads), rotation of the
// first rot dims (dim i with i + rot/2), keys and values into the paged cache.
// One workgroup per token: cos and sin of the token's rot/2 angles are computed
// once into LDS and shared by all heads; then one wave per head at a time, a
// lane owning both dims of a pair, so heads need no exchange between lanes.
// The head row is read twice (statistic, then output): the second read hits L1.
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
  const int half = rot / 2;
  float* cs_s = smem;            // [half]
  float* sn_s = smem + half;     // [half]
  const int tok = blockIdx.x;
  const int lane = threadIdx.x & (WAVE_SIZE - 1);
  const int wave = threadIdx.x / WAVE_SIZE;
  const int nwaves = blockDim.x / WAVE_SIZE;
  const float pos = (float)positions[tok];
  const long slot = slot_mapping[tok];
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    float sn, cs;
    sincosf(pos * inv_freq[i], &sn, &cs);
    cs_s[i] = cs;
    sn_s[i] = sn;
  }
  __syncthreads();
  for (int hh = wave; hh < heads + kv_heads; hh += nwaves) {
    const bool is_q = hh < heads;
    const T* src = is_q ? q + tok * q_st + (long)hh * dim
                        : k + tok * k_st + (long)(hh - heads) * dim;
    T* dst = nullptr;
    if (is_q) dst = q_out + ((long)tok * heads + hh) * dim;
    else if (slot >= 0) dst = k_cache + (slot * kv_heads + (hh - heads)) * dim;
    if (dst == nullptr) continue;
    const float* wt = is_q ? qw : kw;
    float ss = 0.f;
    for (int c = lane; c < dim; c += WAVE_SIZE) {
      const float f = ScalarOps<T>::to_f32(src[c]);
      ss += f * f;
    }
    ss = wave_reduce_sum(ss);
    const float inv = rsqrtf(ss / (float)dim + eps);
    for (int i = lane; i < half; i += WAVE_SIZE) {
      const float a = ScalarOps<T>::to_f32(src[i]) * inv * wt[i];
      const float b = ScalarOps<T>::to_f32(src[i + half]) * inv * wt[i + half];
      const float cs = cs_s[i], sn = sn_s[i];
      dst[i] = ScalarOps<T>::from_f32(a * cs - b * sn);
      dst[i + half] = ScalarOps<T>::from_f32(b * cs + a * sn);
    }
    for (int c = rot + lane; c < dim; c += WAVE_SIZE)
      dst[c] = ScalarOps<T>::from_f32(ScalarOps<T>::to_f32(src[c]) * inv * wt[c]);
  }
  if (slot >= 0) {
    const T* vr = v + tok * v_st;
    T* vd = v_cache + slot * (long)v_heads * vdim;
    for (int c = threadIdx.x; c < v_heads * vdim; c += blockDim.x) vd[c] = vr[c];
  }
}

// The same with 16-byte accesses: eight lanes per head, a lane owning chunks of
// eight consecutive dims, for a rotated pair chunk also its partner chunk, all
// kept in registers between the statistic and the output (one read per input).
// Takes rot/2 and dim - rot in multiples of 8, up to QK_PC pair chunks and
// QK_TC plain chunks per lane.
constexpr int QK_LANES = 8, QK_PC = 2, QK_TC = 2;

template <typename T>
DEVINLINE void load8(const T* p, float* f);
template <>
DEVINLINE void load8<float>(const float* p, float* f) {
  const float4 a = *reinterpret_cast<const float4*>(p);
  const float4 b = *reinterpret_cast<const float4*>(p + 4);
  f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w;
  f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
}
template <>
DEVINLINE void load8<__hip_bfloat16>(const __hip_bfloat16* p, float* f) {
  const uint4 t = *reinterpret_cast<const uint4*>(p);
  const unsigned u[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = __uint_as_float(u[i] << 16);
    f[2 * i + 1] = __uint_as_float(u[i] & 0xffff0000u);
  }
}
template <typename T>
DEVINLINE void store8(T* p, const float* f);
template <>
DEVINLINE void store8<float>(float* p, const float* f) {
  *reinterpret_cast<float4*>(p) = make_float4(f[0], f[1], f[2], f[3]);
  *reinterpret_cast<float4*>(p + 4) = make_float4(f[4], f[5], f[6], f[7]);
}
template <>
DEVINLINE void store8<__hip_bfloat16>(__hip_bfloat16* p, const float* f) {
  union { __hip_bfloat16 h[8]; uint4 u; } o;
#pragma unroll
  for (int i = 0; i < 8; ++i) o.h[i] = __float2bfloat16(f[i]);
  *reinterpret_cast<uint4*>(p) = o.u;
}

template <typename T>
__global__ __launch_bounds__(256) void qk_norm_rope_cache_write_vec_kernel(
    T* __restrict__ q_out, const T* __restrict__ q, long q_st,
    const T* __restrict__ k, long k_st, const T* __restrict__ v, long v_st,
    const float* __restrict__ qw, const float* __restrict__ kw, float eps,
    const long* __restrict__ positions, const float* __restrict__ inv_freq,
    int rot, T* __restrict__ k_cache, T* __restrict__ v_cache,
    const long* __restrict__ slot_mapping, int heads, int kv_heads, int v_heads,
    int dim, int vdim) {
  extern __shared__ float smem[];
  const int half = rot / 2;
  float* cs_s = smem;
  float* sn_s = smem + half;
  const int tok = blockIdx.x;
  const float pos = (float)positions[tok];
  const long slot = slot_mapping[tok];
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    float sn, cs;
    sincosf(pos * inv_freq[i], &sn, &cs);
    cs_s[i] = cs;
    sn_s[i] = sn;
  }
  __syncthreads();
  const int sub = threadIdx.x % QK_LANES;
  const int npc = half / 8, ntc = (dim - rot) / 8;
  const int total = heads + kv_heads;
  const int rounds = (total + 256 / QK_LANES - 1) / (256 / QK_LANES);
  for (int r = 0; r < rounds; ++r) {
    const int hh = r * (256 / QK_LANES) + threadIdx.x / QK_LANES;
    // lanes of a group go together; a group past the last head only joins the
    // shuffles of the reduction
    const bool live = hh < total;
    const bool is_q = hh < heads;
    const T* src = nullptr;
    T* dst = nullptr;
    if (live) {
      src = is_q ? q + tok * q_st + (long)hh * dim : k + tok * k_st + (long)(hh - heads) * dim;
      if (is_q) dst = q_out + ((long)tok * heads + hh) * dim;
      else if (slot >= 0) dst = k_cache + (slot * kv_heads + (hh - heads)) * dim;
    }
    const bool work = dst != nullptr;
    const float* wt = is_q ? qw : kw;
    float pa[QK_PC][8], pb[QK_PC][8], tc[QK_TC][8];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < QK_PC; ++j) {
      const int ch = sub + j * QK_LANES;
      if (work && ch < npc) {
        load8<T>(src + ch * 8, pa[j]);
        load8<T>(src + half + ch * 8, pb[j]);
#pragma unroll
        for (int u = 0; u < 8; ++u) ss += pa[j][u] * pa[j][u] + pb[j][u] * pb[j][u];
      }
    }
#pragma unroll
    for (int j = 0; j < QK_TC; ++j) {
      const int ch = sub + j * QK_LANES;
      if (work && ch < ntc) {
        load8<T>(src + rot + ch * 8, tc[j]);
#pragma unroll
        for (int u = 0; u < 8; ++u) ss += tc[j][u] * tc[j][u];
      }
    }
    ss = group_reduce_sum<QK_LANES>(ss);
    if (!work) continue;
    const float inv = rsqrtf(ss / (float)dim + eps);
#pragma unroll
    for (int j = 0; j < QK_PC; ++j) {
      const int ch = sub + j * QK_LANES;
      if (ch < npc) {
        float oa[8], ob[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int i = ch * 8 + u;
          const float a = pa[j][u] * inv * wt[i];
          const float b = pb[j][u] * inv * wt[i + half];
          const float cs = cs_s[i], sn = sn_s[i];
          oa[u] = a * cs - b * sn;
          ob[u] = b * cs + a * sn;
        }
        store8<T>(dst + ch * 8, oa);
        store8<T>(dst + half + ch * 8, ob);
      }
    }
#pragma unroll
    for (int j = 0; j < QK_TC; ++j) {
      const int ch = sub + j * QK_LANES;
      if (ch < ntc) {
        float o[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) o[u] = tc[j][u] * inv * wt[rot + ch * 8 + u];
        store8<T>(dst + rot + ch * 8, o);
      }
    }
  }
  if (slot >= 0) {
    const T* vr = v + tok * v_st;
    T* vd = v_cache + slot * (long)v_heads * vdim;
    constexpr int E = 16 / sizeof(T);
    const int n = v_heads * vdim;   // the launcher checked n % E == 0 and alignment
    for (int c = threadIdx.x * E; c < n; c += blockDim.x * E)
      *reinterpret_cast<uint4*>(vd + c) = *reinterpret_cast<const uint4*>(vr + c);
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
  constexpr int REG = 4;   // values a lane keeps: rows up to 256 are read once
  float o[REG];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < REG; ++i) {
    const int c = lane + i * WAVE_SIZE;
    o[i] = c < vdim ? a0[c] - lam * a1[c] : 0.f;
    ss += o[i] * o[i];
  }
  for (int c = lane + REG * WAVE_SIZE; c < vdim; c += WAVE_SIZE) {
    const float t2 = a0[c] - lam * a1[c];
    ss += t2 * t2;
  }
  ss = wave_reduce_sum(ss);
  float mul = rsqrtf(ss / (float)vdim + eps) * out_scale;
  if (gate != nullptr) mul *= sigmoid_f(ScalarOps<T>::to_f32(gate[t * g_st + h]));
  T* orow = out + (t * heads + h) * vdim;
#pragma unroll
  for (int i = 0; i < REG; ++i) {
    const int c = lane + i * WAVE_SIZE;
    if (c < vdim) orow[c] = ScalarOps<T>::from_f32(o[i] * mul);
  }
  for (int c = lane + REG * WAVE_SIZE; c < vdim; c += WAVE_SIZE)
    orow[c] = ScalarOps<T>::from_f32((a0[c] - lam * a1[c]) * mul);
}

// ---------------------------------------------------------------------------
// RMS norm of rows in equal groups, times a weight per channel.  Groups of up
// to 256 values: one wave per (row, group), the values kept in registers.
// Longer groups: one workgroup per (row, group).
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
  constexpr int REG = 4;
  float f[REG];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < REG; ++i) {
    const int c = lane + i * WAVE_SIZE;
    f[i] = c < gsize ? ScalarOps<I>::to_f32(yr[c]) : 0.f;
    ss += f[i] * f[i];
  }
  ss = wave_reduce_sum(ss);
  const float inv = rsqrtf(ss / (float)gsize + eps);
  T* orow = out + idx * gsize;
#pragma unroll
  for (int i = 0; i < REG; ++i) {
    const int c = lane + i * WAVE_SIZE;
    if (c < gsize) orow[c] = ScalarOps<T>::from_f32(f[i] * inv * wr[c]);
  }
}

template <typename T, typename I>
__global__ __launch_bounds__(256) void group_rms_norm_wide_kernel(
    T* __restrict__ out, const I* __restrict__ y, const float* __restrict__ w,
    float eps, int groups, int gsize) {
  __shared__ float red[8];
  const long idx = blockIdx.x;
  const int g = (int)(idx % groups);
  const I* yr = y + idx * gsize;
  const float* wr = w + (long)g * gsize;
  float ss = 0.f;
  for (int c = threadIdx.x; c < gsize; c += blockDim.x) {
    const float f = ScalarOps<I>::to_f32(yr[c]);
    ss += f * f;
  }
  ss = block_reduce_sum(ss, red);
  const float inv = rsqrtf(ss / (float)gsize + eps);
  T* orow = out + idx * gsize;
  for (int c = threadIdx.x; c < gsize; c += blockDim.x)
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
  auto al = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  const int vec = width % 4 == 0 && al(out) && al(x) && al(w) && al(state);
  const int per = vec ? 4 : 1;
  const int need = (width + per - 1) / per;
  const int block = need >= 256 ? 256 : ((need + 63) / 64) * 64;
  token_shift_state_kernel<T><<<rows, block, 0, s>>>(out, x, w, state, loc, seq_lens,
                                                    slots, nseq, width, vec);
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
  auto al = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  constexpr int E = 16 / sizeof(T);
  const int half = rot / 2;
  const bool vec = half % 8 == 0 && (dim - rot) % 8 == 0 &&
                   half / 8 <= QK_PC * QK_LANES && (dim - rot) / 8 <= QK_TC * QK_LANES &&
                   q_st % 8 == 0 && k_st % 8 == 0 && v_st % E == 0 &&
                   (v_heads * vdim) % E == 0 && al(q) && al(k) && al(v) && al(q_out) &&
                   al(k_cache) && al(v_cache);
  if (vec) {
    qk_norm_rope_cache_write_vec_kernel<T><<<tokens, 256, sizeof(float) * (rot + 2), s>>>(
        q_out, q, q_st, k, k_st, v, v_st, qw, kw, eps, positions, inv_freq, rot, k_cache,
        v_cache, slot_mapping, heads, kv_heads, v_heads, dim, vdim);
    return;
  }
  const int waves = 4;
  qk_norm_rope_cache_write_kernel<T>
      <<<tokens, waves * WAVE_SIZE, sizeof(float) * (rot + 2), s>>>(
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
  if (gsize <= 4 * WAVE_SIZE)
    group_rms_norm_kernel<T, I><<<(int)((n + 3) / 4), 256, 0, s>>>(out, y, w, eps, rows,
                                                                 groups, gsize);
  else
    group_rms_norm_wide_kernel<T, I><<<(int)n, 256, 0, s>>>(out, y, w, eps, groups, gsize);
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
