// Kernels of parallel two-norm blocks with gated attention and routed experts.
//
//   stream_add_rms_norm_pair  x += a + b + s[row] * c, then the two RMS norms of
//                             the updated row that share one statistic
//   rope_kv_cache_write       rotate queries and keys (half-split or interleaved
//                             pairs, f32 angles, scaled cos/sin), write rotated
//                             keys and the values into the paged cache
//   sigmoid_gate_mul          heads times sigmoid(gate), per element or per head,
//                             regrouping a head-major input to token-major
//   relu2                     relu(x + bias)^2, optionally times a factor per
//                             (row, block of columns)
//   moe_route                 softmax over experts, corrected top-k choice,
//                             normalised weights, identity experts summed
//   moe_combine               weighted gather-sum of expert outputs per token
//   moe_sort                  token-expert pairs grouped by expert: segment
//                             offsets, each pair's row, the gathered input rows
//
// All memory-bound; norm statistics, angles, sigmoids, router arithmetic and
// the stream are f32 whatever the storage type.

#include "common.h"

namespace {

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

template <typename P>
inline bool al(const P* p, size_t bytes) {
  return p == nullptr || reinterpret_cast<uintptr_t>(p) % bytes == 0;
}

inline int grid_for(long n, int block) {
  long g = (n + block - 1) / block;
  return (int)(g < 1 ? 1 : (g > 65535 ? 65535 : g));
}

DEVINLINE float sigmoid_f32(float z) { return 1.0f / (1.0f + expf(-z)); }

// One workgroup per row.  Pass 1 forms the new row (when `a` is given) and its
// sum of squares; pass 2 re-reads what each thread wrote itself and stores the
// two normed rows.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void stream_add_rms_norm_pair_kernel(
    float* __restrict__ x, const T* __restrict__ a, const T* __restrict__ b,
    const float* __restrict__ row_scale, const T* __restrict__ c,
    const float* __restrict__ w1, const float* __restrict__ w2, float eps,
    int width, T* __restrict__ h1, T* __restrict__ h2) {
  const long row = blockIdx.x;
  float* xr = x + row * width;
  const long off = row * width;
  constexpr int S = VEC ? 4 : 1;
  const float rs = (c != nullptr) ? row_scale[row] : 0.f;
  float ss = 0.f;
  for (int k = threadIdx.x * S; k < width; k += blockDim.x * S) {
    if (VEC) {
      F4 v = Pack4<float>::load(xr + k);
      if (a != nullptr) {
        F4 s = Pack4<T>::load(a + off + k);
        if (b != nullptr) {
          const F4 t = Pack4<T>::load(b + off + k);
#pragma unroll
          for (int i = 0; i < 4; ++i) s.v[i] += t.v[i];
        }
        if (c != nullptr) {
          const F4 t = Pack4<T>::load(c + off + k);
#pragma unroll
          for (int i = 0; i < 4; ++i) s.v[i] += rs * t.v[i];
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) v.v[i] += s.v[i];
        Pack4<float>::store(xr + k, v);
      }
      ss += (v.v[0] * v.v[0] + v.v[1] * v.v[1]) + (v.v[2] * v.v[2] + v.v[3] * v.v[3]);
    } else {
      float v = xr[k];
      if (a != nullptr) {
        float s = ScalarOps<T>::to_f32(a[off + k]);
        if (b != nullptr) s += ScalarOps<T>::to_f32(b[off + k]);
        if (c != nullptr) s += rs * ScalarOps<T>::to_f32(c[off + k]);
        v += s;
        xr[k] = v;
      }
      ss += v * v;
    }
  }
  if (w1 == nullptr && w2 == nullptr) return;
  __shared__ float lds[16];
  ss = block_reduce_sum(ss, lds);
  const float inv = 1.0f / sqrtf(ss / width + eps);
  for (int k = threadIdx.x * S; k < width; k += blockDim.x * S) {
    if (VEC) {
      const F4 v = Pack4<float>::load(xr + k);
      if (w1 != nullptr) {
        const F4 g = Pack4<float>::load(w1 + k);
        F4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o.v[i] = v.v[i] * inv * g.v[i];
        Pack4<T>::store(h1 + off + k, o);
      }
      if (w2 != nullptr) {
        const F4 g = Pack4<float>::load(w2 + k);
        F4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o.v[i] = v.v[i] * inv * g.v[i];
        Pack4<T>::store(h2 + off + k, o);
      }
    } else {
      const float v = xr[k] * inv;
      if (w1 != nullptr) h1[off + k] = ScalarOps<T>::from_f32(v * w1[k]);
      if (w2 != nullptr) h2[off + k] = ScalarOps<T>::from_f32(v * w2[k]);
    }
  }
}

// One wave per (token, unit): units 0..H-1 are query heads (rotated into
// q_out), H..H+G-1 key heads (rotated into the key cache), H+G..H+2G-1 value
// heads (copied into the value cache).  Element c < 2*half of a rotated head is
// x[c] cos + (c is the pair's first ? -x[partner] : x[partner]) sin.
template <typename T>
__global__ __launch_bounds__(256) void rope_kv_cache_write_kernel(
    T* __restrict__ q_out, const T* __restrict__ q, long q_st,
    const T* __restrict__ k, long k_st, const T* __restrict__ v, long v_st,
    const long* __restrict__ positions, const float* __restrict__ inv_freq,
    int half, int interleaved, float mag, T* __restrict__ k_cache,
    T* __restrict__ v_cache, const long* __restrict__ slot_mapping, int heads,
    int kv_heads, int dim, int vdim) {
  const long t = blockIdx.x;
  const int lane = threadIdx.x & (WAVE_SIZE - 1);
  const int unit = blockIdx.y * (blockDim.x / WAVE_SIZE) + threadIdx.x / WAVE_SIZE;
  if (unit >= heads + 2 * kv_heads) return;
  const long slot = slot_mapping[t];
  if (unit >= heads + kv_heads) {
    if (slot < 0) return;
    const int g = unit - heads - kv_heads;
    const T* src = v + t * v_st + (long)g * vdim;
    T* dst = v_cache + (slot * kv_heads + g) * vdim;
    for (int c = lane; c < vdim; c += WAVE_SIZE) dst[c] = src[c];
    return;
  }
  const bool is_q = unit < heads;
  const int hh = is_q ? unit : unit - heads;
  if (!is_q && slot < 0) return;
  const T* src = is_q ? q + t * q_st + (long)hh * dim : k + t * k_st + (long)hh * dim;
  T* dst = is_q ? q_out + (t * heads + hh) * dim : k_cache + (slot * kv_heads + hh) * dim;
  const float pos = (float)positions[t];
  const int rot = 2 * half;
  for (int c = lane; c < dim; c += WAVE_SIZE) {
    if (c >= rot) {
      dst[c] = src[c];
      continue;
    }
    int pair, partner;
    bool first;
    if (interleaved) {
      pair = c >> 1;
      partner = c ^ 1;
      first = (c & 1) == 0;
    } else {
      first = c < half;
      pair = first ? c : c - half;
      partner = first ? c + half : c - half;
    }
    float sn, cs;
    sincosf(pos * inv_freq[pair], &sn, &cs);
    sn *= mag;
    cs *= mag;
    const float self = ScalarOps<T>::to_f32(src[c]);
    const float other = ScalarOps<T>::to_f32(src[partner]);
    dst[c] = ScalarOps<T>::from_f32(first ? self * cs - other * sn : self * cs + other * sn);
  }
}

// Vector variant: `lph` lanes per head, each owning 16 bytes (V elements) of
// it; sizes and strides are multiples of V, for half-split pairs the half is a
// multiple of V too (the lane of the first half also loads, rotates and stores
// the partner chunk).  grid (tokens, ceil(units / units_per_block)).
template <typename T>
__global__ __launch_bounds__(256) void rope_kv_cache_write_vec_kernel(
    T* __restrict__ q_out, const T* __restrict__ q, long q_st,
    const T* __restrict__ k, long k_st, const T* __restrict__ v, long v_st,
    const long* __restrict__ positions, const float* __restrict__ inv_freq,
    int half, int interleaved, float mag, T* __restrict__ k_cache,
    T* __restrict__ v_cache, const long* __restrict__ slot_mapping, int heads,
    int kv_heads, int dim, int vdim, int lph, int upb) {
  constexpr int V = Vec16<T>::kElems;
  const long t = blockIdx.x;
  const int u_in = threadIdx.x / lph;
  const int l = threadIdx.x - u_in * lph;
  const int unit = blockIdx.y * upb + u_in;
  if (u_in >= upb || unit >= heads + 2 * kv_heads) return;
  const long slot = slot_mapping[t];
  const int c0 = l * V;
  if (unit >= heads + kv_heads) {
    if (slot < 0 || c0 >= vdim) return;
    const int g = unit - heads - kv_heads;
    store16(v_cache + (slot * kv_heads + g) * vdim + c0,
            load16(v + t * v_st + (long)g * vdim + c0));
    return;
  }
  if (c0 >= dim) return;
  const bool is_q = unit < heads;
  const int hh = is_q ? unit : unit - heads;
  if (!is_q && slot < 0) return;
  const T* src = is_q ? q + t * q_st + (long)hh * dim : k + t * k_st + (long)hh * dim;
  T* dst = is_q ? q_out + (t * heads + hh) * dim : k_cache + (slot * kv_heads + hh) * dim;
  const int rot = 2 * half;
  Vec16<T> a = load16(src + c0);
  if (c0 >= rot) {
    store16(dst + c0, a);
    return;
  }
  const float pos = (float)positions[t];
  if (interleaved) {
#pragma unroll
    for (int i = 0; i < V / 2; ++i) {
      float sn, cs;
      sincosf(pos * inv_freq[c0 / 2 + i], &sn, &cs);
      sn *= mag;
      cs *= mag;
      const float x0 = ScalarOps<T>::to_f32(a.data[2 * i]);
      const float x1 = ScalarOps<T>::to_f32(a.data[2 * i + 1]);
      a.data[2 * i] = ScalarOps<T>::from_f32(x0 * cs - x1 * sn);
      a.data[2 * i + 1] = ScalarOps<T>::from_f32(x1 * cs + x0 * sn);
    }
    store16(dst + c0, a);
    return;
  }
  if (c0 >= half) return;   // written by the lane that owns the first half
  Vec16<T> b = load16(src + c0 + half);
#pragma unroll
  for (int i = 0; i < V; ++i) {
    float sn, cs;
    sincosf(pos * inv_freq[c0 + i], &sn, &cs);
    sn *= mag;
    cs *= mag;
    const float x0 = ScalarOps<T>::to_f32(a.data[i]);
    const float x1 = ScalarOps<T>::to_f32(b.data[i]);
    a.data[i] = ScalarOps<T>::from_f32(x0 * cs - x1 * sn);
    b.data[i] = ScalarOps<T>::from_f32(x1 * cs + x0 * sn);
  }
  store16(dst + c0, a);
  store16(dst + c0 + half, b);
}

// out[t, h*D + d] = o[t, h, d] * sigmoid(gate); n counts groups of S elements.
template <typename T, bool VEC>
__global__ void sigmoid_gate_mul_kernel(T* __restrict__ out, const T* __restrict__ o,
                                        long o_st, long o_sh,
                                        const T* __restrict__ gate, long g_st,
                                        long g_sh, int per_head, int heads, int d,
                                        long n) {
  constexpr int S = VEC ? 4 : 1;
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n;
       i += (long)gridDim.x * blockDim.x) {
    const long e = i * S;
    const int dd = (int)(e % d);
    const long th = e / d;
    const int h = (int)(th % heads);
    const long t = th / heads;
    const T* op = o + t * o_st + h * o_sh + dd;
    if (VEC) {
      F4 f = Pack4<T>::load(op);
      if (per_head) {
        const float g = sigmoid_f32(ScalarOps<T>::to_f32(gate[t * g_st + h]));
#pragma unroll
        for (int k = 0; k < 4; ++k) f.v[k] *= g;
      } else {
        const F4 g = Pack4<T>::load(gate + t * g_st + h * g_sh + dd);
#pragma unroll
        for (int k = 0; k < 4; ++k) f.v[k] *= sigmoid_f32(g.v[k]);
      }
      Pack4<T>::store(out + e, f);
    } else {
      const float g = per_head ? ScalarOps<T>::to_f32(gate[t * g_st + h])
                               : ScalarOps<T>::to_f32(gate[t * g_st + h * g_sh + dd]);
      out[e] = ScalarOps<T>::from_f32(ScalarOps<T>::to_f32(*op) * sigmoid_f32(g));
    }
  }
}

// out = relu(x + bias[col])^2 [* col_scale[row, col / per]]
template <typename T, bool VEC>
__global__ void relu2_kernel(T* __restrict__ out, const T* __restrict__ x,
                             long x_st, const T* __restrict__ bias,
                             const float* __restrict__ col_scale, int nscale,
                             int per, int cols, long n) {
  constexpr int S = VEC ? 4 : 1;
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n;
       i += (long)gridDim.x * blockDim.x) {
    const long e = i * S;
    const long r = e / cols;
    const int c = (int)(e - r * cols);
    const float sc = (col_scale != nullptr) ? col_scale[r * nscale + c / per] : 1.0f;
    if (VEC) {
      F4 f = Pack4<T>::load(x + r * x_st + c);
      if (bias != nullptr) {
        const F4 bb = Pack4<T>::load(bias + c);
#pragma unroll
        for (int k = 0; k < 4; ++k) f.v[k] += bb.v[k];
      }
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float z = fmaxf(f.v[k], 0.f);
        f.v[k] = z * z * sc;
      }
      Pack4<T>::store(out + e, f);
    } else {
      float z = ScalarOps<T>::to_f32(x[r * x_st + c]);
      if (bias != nullptr) z += ScalarOps<T>::to_f32(bias[c]);
      z = fmaxf(z, 0.f);
      out[e] = ScalarOps<T>::from_f32(z * z * sc);
    }
  }
}

// One wave per token; lane l owns experts l, l + 64, ... (at most RT_MAX each).
constexpr int RT_MAX = 8;

__global__ __launch_bounds__(256) void moe_route_kernel(
    float* __restrict__ dense, float* __restrict__ ident, int* __restrict__ ids,
    float* __restrict__ wts, const float* __restrict__ logits,
    const float* __restrict__ correction, int tokens, int n, int num_real,
    int top, int sigmoid) {
  // sigmoid: scores are sigmoid(logit) instead of the softmax, there is no
  // correction (nullptr), no identity output and no renormalising
  const int lane = threadIdx.x & (WAVE_SIZE - 1);
  const long t = blockIdx.x * (long)(blockDim.x / WAVE_SIZE) + threadIdx.x / WAVE_SIZE;
  if (t >= tokens) return;
  const float* z = logits + t * n;
  float s[RT_MAX], ch[RT_MAX];
  bool taken[RT_MAX];
  float m = -INFINITY;
#pragma unroll
  for (int i = 0; i < RT_MAX; ++i) {
    const int e = lane + i * WAVE_SIZE;
    s[i] = (e < n) ? z[e] : -INFINITY;
    taken[i] = false;
    m = fmaxf(m, s[i]);
  }
  if (sigmoid) {
#pragma unroll
    for (int i = 0; i < RT_MAX; ++i) {
      const int e = lane + i * WAVE_SIZE;
      s[i] = (e < n) ? 1.0f / (1.0f + expf(-s[i])) : 0.f;
      ch[i] = (e < n) ? s[i] : -INFINITY;
    }
  } else {
    m = wave_reduce_max(m);
    float den = 0.f;
#pragma unroll
    for (int i = 0; i < RT_MAX; ++i) {
      const int e = lane + i * WAVE_SIZE;
      s[i] = (e < n) ? expf(s[i] - m) : 0.f;
      den += s[i];
    }
    den = wave_reduce_sum(den);
#pragma unroll
    for (int i = 0; i < RT_MAX; ++i) {
      const int e = lane + i * WAVE_SIZE;
      s[i] = s[i] / den;
      ch[i] = (e < n) ? s[i] + correction[e] : -INFINITY;
    }
  }
  float total = 0.f, id_sum = 0.f;
  for (int k = 0; k < top; ++k) {
    // the largest remaining choice score; ties go to the lower index
    float best = -INFINITY;
    int best_e = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < RT_MAX; ++i) {
      const int e = lane + i * WAVE_SIZE;
      if (e < n && !taken[i] && (ch[i] > best || (ch[i] == best && e < best_e))) {
        best = ch[i];
        best_e = e;
      }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, WAVE_SIZE);
      const int oe = __shfl_xor(best_e, off, WAVE_SIZE);
      if (ob > best || (ob == best && oe < best_e)) {
        best = ob;
        best_e = oe;
      }
    }
    // the owner marks it and tells everyone its softmax score
    float sv = 0.f;
#pragma unroll
    for (int i = 0; i < RT_MAX; ++i) {
      if (lane + i * WAVE_SIZE == best_e) {
        taken[i] = true;
        sv = s[i];
      }
    }
    sv = wave_reduce_sum(sv);
    total += sv;
    if (best_e >= num_real) id_sum += sv;
    if (lane == 0) {
      ids[t * top + k] = best_e;
      wts[t * top + k] = sv;
    }
  }
  const float inv = sigmoid ? 1.0f : 1.0f / (total + 1e-20f);
#pragma unroll
  for (int i = 0; i < RT_MAX; ++i) {
    const int e = lane + i * WAVE_SIZE;
    if (e < num_real) dense[t * num_real + e] = taken[i] ? s[i] * inv : 0.f;
  }
  // lane 0 wrote wts[t, :] itself, so it may rescale them in place
  if (lane == 0 && !sigmoid) {
    for (int k = 0; k < top; ++k) wts[t * top + k] *= inv;
    ident[t] = id_sum * inv;
  }
}

// out[t, :] = sum_k [ids[t,k] < num_real] w[t,k] * ye[pos[t,k], :]
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void moe_combine_kernel(
    T* __restrict__ out, const T* __restrict__ ye, const int* __restrict__ pos,
    const int* __restrict__ ids, const float* __restrict__ wts, int top,
    int num_real, int width) {
  const long t = blockIdx.x;
  constexpr int S = VEC ? 4 : 1;
  for (int c = threadIdx.x * S; c < width; c += blockDim.x * S) {
    F4 acc{{0.f, 0.f, 0.f, 0.f}};
    for (int k = 0; k < top; ++k) {
      if (ids[t * top + k] >= num_real) continue;
      const float w = wts[t * top + k];
      const T* src = ye + (long)pos[t * top + k] * width + c;
      if (VEC) {
        const F4 f = Pack4<T>::load(src);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc.v[i] += w * f.v[i];
      } else {
        acc.v[0] += w * ScalarOps<T>::to_f32(*src);
      }
    }
    if (VEC) Pack4<T>::store(out + t * width + c, acc);
    else out[t * width + c] = ScalarOps<T>::from_f32(acc.v[0]);
  }
}

// Grouping token-expert pairs by expert without a sort: count the pairs of
// each real expert, turn the counts into segment offsets, hand every pair the
// next free row of its expert's segment, copy the token's input row there.
// Which row of its segment a pair gets depends on the order the atomics land
// in; the grouped product computes every row on its own, so the values do not.
constexpr int MS_MAX = 512;   // real experts

__global__ __launch_bounds__(256) void moe_count_kernel(
    int* __restrict__ counts, const int* __restrict__ ids, int npairs, int num_real) {
  __shared__ int hist[MS_MAX];
  for (int e = threadIdx.x; e < num_real; e += blockDim.x) hist[e] = 0;
  __syncthreads();
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < npairs;
       i += gridDim.x * blockDim.x) {
    const int e = ids[i];
    if (e < num_real) atomicAdd(&hist[e], 1);
  }
  __syncthreads();
  for (int e = threadIdx.x; e < num_real; e += blockDim.x)
    if (hist[e]) atomicAdd(&counts[e], hist[e]);
}

__global__ __launch_bounds__(256) void moe_place_kernel(
    int* __restrict__ pos, int* __restrict__ seg, int* __restrict__ cursor,
    const int* __restrict__ counts, const int* __restrict__ ids, int npairs,
    int num_real) {
  __shared__ int seg_s[MS_MAX + 1];
  __shared__ int hist[MS_MAX];   // the workgroup's pairs of this pass, per expert
  __shared__ int base[MS_MAX];   // where the workgroup's run starts in the segment
  if (threadIdx.x == 0) {
    int run = 0;
    for (int e = 0; e < num_real; ++e) {
      seg_s[e] = run;
      run += counts[e];
    }
    seg_s[num_real] = run;
  }
  __syncthreads();
  if (blockIdx.x == 0)
    for (int e = threadIdx.x; e <= num_real; e += blockDim.x) seg[e] = seg_s[e];
  // passes of one pair per thread: rank the pairs inside the workgroup through
  // LDS, reserve one run per (workgroup, expert) with a single global atomic
  const int stride = gridDim.x * blockDim.x;
  const int passes = (npairs + stride - 1) / stride;
  for (int r = 0; r < passes; ++r) {
    const int i = r * stride + blockIdx.x * blockDim.x + threadIdx.x;
    for (int e = threadIdx.x; e < num_real; e += blockDim.x) hist[e] = 0;
    __syncthreads();
    int e = num_real, local = 0;
    if (i < npairs) {
      e = ids[i];
      if (e < num_real) local = atomicAdd(&hist[e], 1);
    }
    __syncthreads();
    for (int x = threadIdx.x; x < num_real; x += blockDim.x)
      if (hist[x]) base[x] = atomicAdd(&cursor[x], hist[x]);
    __syncthreads();
    if (i < npairs) pos[i] = (e < num_real) ? seg_s[e] + base[e] + local : 0;
    __syncthreads();   // hist and base are reused by the next pass
  }
}

// one workgroup per token: its row goes to the rows of its real experts
template <typename T>
__global__ __launch_bounds__(256) void moe_gather_kernel(
    T* __restrict__ xs, const T* __restrict__ h, long h_st,
    const int* __restrict__ pos, const int* __restrict__ ids, int top,
    int num_real, int width, int vec, const float* __restrict__ row_scale) {
  const long t = blockIdx.x;
  const T* src = h + t * h_st;
  if (vec) {
    constexpr int V = Vec16<T>::kElems;
    for (int c = threadIdx.x * V; c < width; c += blockDim.x * V) {
      const Vec16<T> v = load16(src + c);
      for (int k = 0; k < top; ++k) {
        if (ids[t * top + k] >= num_real) continue;
        if (row_scale == nullptr) {
          store16(xs + (long)pos[t * top + k] * width + c, v);
        } else {
          const float sc = row_scale[t * top + k];
          Vec16<T> o;
#pragma unroll
          for (int u = 0; u < V; ++u)
            o.data[u] = ScalarOps<T>::from_f32(ScalarOps<T>::to_f32(v.data[u]) * sc);
          store16(xs + (long)pos[t * top + k] * width + c, o);
        }
      }
    }
  } else {
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
      const T v = src[c];
      for (int k = 0; k < top; ++k) {
        if (ids[t * top + k] >= num_real) continue;
        xs[(long)pos[t * top + k] * width + c] =
            row_scale == nullptr
                ? v
                : ScalarOps<T>::from_f32(ScalarOps<T>::to_f32(v) * row_scale[t * top + k]);
      }
    }
  }
}

}  // namespace

// ---------------------------------------------------------------------------
// launchers
// ---------------------------------------------------------------------------

int moe_sort_max_experts() { return MS_MAX; }

// counts_cursor: 2 * num_real zeros (counts, then the per-expert cursors)
template <typename T>
void launch_moe_sort(T* xs, int* pos, int* seg, int* counts_cursor, const T* h,
                     long h_st, const int* ids, int tokens, int top, int num_real,
                     int width, const float* row_scale, hipStream_t s) {
  const int npairs = tokens * top;
  const int blocks = grid_for(npairs, 256) > 1024 ? 1024 : grid_for(npairs, 256);
  moe_count_kernel<<<blocks, 256, 0, s>>>(counts_cursor, ids, npairs, num_real);
  moe_place_kernel<<<blocks, 256, 0, s>>>(pos, seg, counts_cursor + num_real,
                                           counts_cursor, ids, npairs, num_real);
  constexpr int V = Vec16<T>::kElems;
  const int vec = width % V == 0 && h_st % V == 0 && al(xs, 16) && al(h, 16);
  moe_gather_kernel<T><<<tokens, 256, 0, s>>>(xs, h, h_st, pos, ids, top, num_real,
                                             width, vec, row_scale);
}

template <typename T>
void launch_stream_add_rms_norm_pair(float* x, const T* a, const T* b,
                                     const float* row_scale, const T* c,
                                     const float* w1, const float* w2, float eps,
                                     int rows, int width, T* h1, T* h2,
                                     hipStream_t s) {
  const size_t tb = 4 * sizeof(T);
  if (width % 4 == 0 && al(x, 16) && al(a, tb) && al(b, tb) && al(c, tb) &&
      al(w1, 16) && al(w2, 16) && al(h1, tb) && al(h2, tb))
    stream_add_rms_norm_pair_kernel<T, true><<<rows, 256, 0, s>>>(
        x, a, b, row_scale, c, w1, w2, eps, width, h1, h2);
  else
    stream_add_rms_norm_pair_kernel<T, false><<<rows, 256, 0, s>>>(
        x, a, b, row_scale, c, w1, w2, eps, width, h1, h2);
}

template <typename T>
void launch_rope_kv_cache_write(T* q_out, const T* q, long q_st, const T* k,
                                long k_st, const T* v, long v_st,
                                const long* positions, const float* inv_freq,
                                int half, int interleaved, float mag, T* k_cache,
                                T* v_cache, const long* slot_mapping, int tokens,
                                int heads, int kv_heads, int dim, int vdim,
                                hipStream_t s) {
  const int units = heads + 2 * kv_heads;
  constexpr int V = Vec16<T>::kElems;
  const int rot = 2 * half;
  const int big = dim > vdim ? dim : vdim;
  const bool vec = dim % V == 0 && vdim % V == 0 && big / V <= 256 && q_st % V == 0 &&
                   k_st % V == 0 && v_st % V == 0 && rot % V == 0 &&
                   (interleaved || half % V == 0) && al(q_out, 16) && al(q, 16) &&
                   al(k, 16) && al(v, 16) && al(k_cache, 16) && al(v_cache, 16);
  if (vec) {
    const int lph = big / V;
    const int upb = 256 / lph;
    dim3 vgrid(tokens, (units + upb - 1) / upb);
    rope_kv_cache_write_vec_kernel<T><<<vgrid, 256, 0, s>>>(
        q_out, q, q_st, k, k_st, v, v_st, positions, inv_freq, half, interleaved,
        mag, k_cache, v_cache, slot_mapping, heads, kv_heads, dim, vdim, lph, upb);
    return;
  }
  dim3 grid(tokens, (units + 3) / 4);
  rope_kv_cache_write_kernel<T><<<grid, 256, 0, s>>>(
      q_out, q, q_st, k, k_st, v, v_st, positions, inv_freq, half, interleaved,
      mag, k_cache, v_cache, slot_mapping, heads, kv_heads, dim, vdim);
}

template <typename T>
void launch_sigmoid_gate_mul(T* out, const T* o, long o_st, long o_sh,
                             const T* gate, long g_st, long g_sh, int per_head,
                             int tokens, int heads, int d, hipStream_t s) {
  const long n = (long)tokens * heads * d;
  const size_t tb = 4 * sizeof(T);
  const bool vec = d % 4 == 0 && o_st % 4 == 0 && o_sh % 4 == 0 && al(out, tb) &&
                   al(o, tb) &&
                   (per_head || (g_st % 4 == 0 && g_sh % 4 == 0 && al(gate, tb)));
  if (vec)
    sigmoid_gate_mul_kernel<T, true><<<grid_for(n / 4, 256), 256, 0, s>>>(
        out, o, o_st, o_sh, gate, g_st, g_sh, per_head, heads, d, n / 4);
  else
    sigmoid_gate_mul_kernel<T, false><<<grid_for(n, 256), 256, 0, s>>>(
        out, o, o_st, o_sh, gate, g_st, g_sh, per_head, heads, d, n);
}

template <typename T>
void launch_relu2(T* out, const T* x, long x_st, const T* bias,
                  const float* col_scale, int nscale, int rows, int cols,
                  hipStream_t s) {
  const long n = (long)rows * cols;
  const int per = nscale > 0 ? cols / nscale : cols;
  const size_t tb = 4 * sizeof(T);
  const bool vec = cols % 4 == 0 && x_st % 4 == 0 && per % 4 == 0 && al(out, tb) &&
                   al(x, tb) && al(bias, tb);
  if (vec)
    relu2_kernel<T, true><<<grid_for(n / 4, 256), 256, 0, s>>>(
        out, x, x_st, bias, col_scale, nscale, per, cols, n / 4);
  else
    relu2_kernel<T, false><<<grid_for(n, 256), 256, 0, s>>>(
        out, x, x_st, bias, col_scale, nscale, per, cols, n);
}

int moe_route_max_experts() { return RT_MAX * WAVE_SIZE; }

void launch_moe_route(float* dense, float* ident, int* ids, float* wts,
                      const float* logits, const float* correction, int tokens,
                      int n, int num_real, int top, int sigmoid, hipStream_t s) {
  const int waves = 256 / WAVE_SIZE;
  moe_route_kernel<<<(tokens + waves - 1) / waves, 256, 0, s>>>(
      dense, ident, ids, wts, logits, correction, tokens, n, num_real, top, sigmoid);
}

template <typename T>
void launch_moe_combine(T* out, const T* ye, const int* pos, const int* ids,
                        const float* wts, int tokens, int top, int num_real,
                        int width, hipStream_t s) {
  if (width % 4 == 0 && al(out, 4 * sizeof(T)) && al(ye, 4 * sizeof(T)))
    moe_combine_kernel<T, true><<<tokens, 256, 0, s>>>(out, ye, pos, ids, wts, top,
                                                       num_real, width);
  else
    moe_combine_kernel<T, false><<<tokens, 256, 0, s>>>(out, ye, pos, ids, wts, top,
                                                        num_real, width);
}

#define INSTANTIATE(T)                                                           \
  template void launch_moe_sort<T>(T*, int*, int*, int*, const T*, long,         \
                                   const int*, int, int, int, int, const float*, \
                                   hipStream_t);                                 \
  template void launch_stream_add_rms_norm_pair<T>(                              \
      float*, const T*, const T*, const float*, const T*, const float*,          \
      const float*, float, int, int, T*, T*, hipStream_t);                       \
  template void launch_rope_kv_cache_write<T>(                                   \
      T*, const T*, long, const T*, long, const T*, long, const long*,           \
      const float*, int, int, float, T*, T*, const long*, int, int, int, int,    \
      int, hipStream_t);                                                         \
  template void launch_sigmoid_gate_mul<T>(T*, const T*, long, long, const T*,   \
                                           long, long, int, int, int, int,       \
                                           hipStream_t);                         \
  template void launch_relu2<T>(T*, const T*, long, const T*, const float*, int, \
                                int, int, hipStream_t);                          \
  template void launch_moe_combine<T>(T*, const T*, const int*, const int*,      \
                                      const float*, int, int, int, int,          \
                                      hipStream_t);
INSTANTIATE(float)
INSTANTIATE(__hip_bfloat16)
