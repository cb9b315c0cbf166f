// Ops around an f32 residual stream.
//
// Models that keep their residual in f32 read it through an RMS norm into the
// compute dtype (bf16 or f32), run projections there, and add the results back
// in f32.  All of these are memory-bound row or elementwise kernels: one
// workgroup per row for the norms (sum of squares in f32, block reduce), grid
// stride loops otherwise.  Rotation angles, norm statistics and the stream
// itself never leave f32.

#include "common.h"

// 4-element accessors: 16-byte f32 / 8-byte bf16 accesses when the row length
// is a multiple of 4 (every row then starts 4-aligned), scalar tail otherwise.
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

DEVINLINE float gelu_tanh_f32(float z) {
  const float k = 0.7978845608028654f;  // sqrt(2/pi)
  return 0.5f * z * (1.0f + tanhf(k * (z + 0.044715f * z * z * z)));
}

// out = gelu_tanh(x) [* mul]; x and mul rows may be strided (column slices).
// VEC: cols and the strides are multiples of 4, n counts groups of 4.
template <typename T, bool VEC>
__global__ void gelu_tanh_kernel(T* __restrict__ out, const T* __restrict__ x,
                                 long x_stride, const T* __restrict__ mul,
                                 long mul_stride, int cols, long n) {
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n;
       i += (long)gridDim.x * blockDim.x) {
    if (VEC) {
      const long e = i * 4;
      const long r = e / cols;
      F4 f = Pack4<T>::load(x + r * x_stride + (e - r * cols));
#pragma unroll
      for (int k = 0; k < 4; ++k) f.v[k] = gelu_tanh_f32(f.v[k]);
      if (mul != nullptr) {
        const F4 m = Pack4<T>::load(mul + r * mul_stride + (e - r * cols));
#pragma unroll
        for (int k = 0; k < 4; ++k) f.v[k] *= m.v[k];
      }
      Pack4<T>::store(out + e, f);
    } else {
      const long r = i / cols;
      const int c = (int)(i - r * cols);
      float y = gelu_tanh_f32(ScalarOps<T>::to_f32(x[r * x_stride + c]));
      if (mul != nullptr) y *= ScalarOps<T>::to_f32(mul[r * mul_stride + c]);
      out[i] = ScalarOps<T>::from_f32(y);
    }
  }
}

// out[t, :] = float(table[ids[t], :]) * scale
template <typename T>
__global__ void embedding_scaled_kernel(float* __restrict__ out,
                                        const long* __restrict__ ids,
                                        const T* __restrict__ table,
                                        float scale, int width) {
  const long t = blockIdx.x;
  const T* row = table + ids[t] * (long)width;
  for (int c = threadIdx.x; c < width; c += blockDim.x)
    out[t * width + c] = ScalarOps<T>::to_f32(row[c]) * scale;
}

// out = x / sqrt(mean(x^2) + eps) * (offset + w), x and w f32
template <typename T, bool VEC>
__global__ void rms_norm_stream_kernel(T* __restrict__ out,
                                       const float* __restrict__ x,
                                       const float* __restrict__ w, float eps,
                                       float offset, int width) {
  const long row = blockIdx.x;
  const float* xr = x + row * width;
  constexpr int S = VEC ? 4 : 1;
  float ss = 0.f;
  for (int c = threadIdx.x * S; c < width; c += blockDim.x * S) {
    if (VEC) {
      const F4 f = Pack4<float>::load(xr + c);
      ss += f.v[0] * f.v[0] + f.v[1] * f.v[1] + f.v[2] * f.v[2] + f.v[3] * f.v[3];
    } else {
      ss += xr[c] * xr[c];
    }
  }
  __shared__ float lds[16];
  ss = block_reduce_sum(ss, lds);
  const float inv = 1.0f / sqrtf(ss / width + eps);
  for (int c = threadIdx.x * S; c < width; c += blockDim.x * S) {
    if (VEC) {
      F4 f = Pack4<float>::load(xr + c);
      const F4 g = Pack4<float>::load(w + c);
#pragma unroll
      for (int k = 0; k < 4; ++k) f.v[k] = f.v[k] * inv * (offset + g.v[k]);
      Pack4<T>::store(out + row * width + c, f);
    } else {
      out[row * width + c] = ScalarOps<T>::from_f32(xr[c] * inv * (offset + w[c]));
    }
  }
}

// x += mult * (a + b); cast = T(x) when asked for.  VEC: n counts groups of 4.
template <typename T, bool VEC>
__global__ void stream_add_kernel(float* __restrict__ x, const T* __restrict__ a,
                                  const T* __restrict__ b, float mult,
                                  T* __restrict__ cast, long n) {
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n;
       i += (long)gridDim.x * blockDim.x) {
    if (VEC) {
      const long e = i * 4;
      F4 s = Pack4<T>::load(a + e);
      if (b != nullptr) {
        const F4 t = Pack4<T>::load(b + e);
#pragma unroll
        for (int k = 0; k < 4; ++k) s.v[k] += t.v[k];
      }
      F4 v = Pack4<float>::load(x + e);
#pragma unroll
      for (int k = 0; k < 4; ++k) v.v[k] += mult * s.v[k];
      Pack4<float>::store(x + e, v);
      if (cast != nullptr) Pack4<T>::store(cast + e, v);
    } else {
      float s = ScalarOps<T>::to_f32(a[i]);
      if (b != nullptr) s += ScalarOps<T>::to_f32(b[i]);
      const float v = x[i] + mult * s;
      x[i] = v;
      if (cast != nullptr) cast[i] = ScalarOps<T>::from_f32(v);
    }
  }
}

// x += mult * y / sqrt(mean(y^2) + eps) * w; with next_w also the following
// norm of the updated row: next_out = x / sqrt(mean(x^2) + next_eps) *
// (next_offset + next_w) — the stream is read once for both.
template <typename T, bool VEC>
__global__ void stream_add_rms_norm_kernel(float* __restrict__ x,
                                           const T* __restrict__ y,
                                           const float* __restrict__ w,
                                           float eps, float mult, int width,
                                           T* __restrict__ next_out,
                                           const float* __restrict__ next_w,
                                           float next_eps, float next_offset,
                                           const float* __restrict__ ls) {
  // ls: optional per-channel layer scale on the normed rows.  next_out without
  // next_w: the updated stream rounded to T, no norm.
  const long row = blockIdx.x;
  const T* yr = y + row * width;
  float* xr = x + row * width;
  constexpr int S = VEC ? 4 : 1;
  float ss = 0.f;
  for (int c = threadIdx.x * S; c < width; c += blockDim.x * S) {
    if (VEC) {
      const F4 f = Pack4<T>::load(yr + c);
      ss += f.v[0] * f.v[0] + f.v[1] * f.v[1] + f.v[2] * f.v[2] + f.v[3] * f.v[3];
    } else {
      const float v = ScalarOps<T>::to_f32(yr[c]);
      ss += v * v;
    }
  }
  __shared__ float lds[16];
  ss = block_reduce_sum(ss, lds);
  const float inv = 1.0f / sqrtf(ss / width + eps);
  float sx = 0.f;
  for (int c = threadIdx.x * S; c < width; c += blockDim.x * S) {
    if (VEC) {
      const F4 f = Pack4<T>::load(yr + c);
      const F4 g = Pack4<float>::load(w + c);
      F4 v = Pack4<float>::load(xr + c);
      if (ls != nullptr) {
        const F4 l = Pack4<float>::load(ls + c);
#pragma unroll
        for (int k = 0; k < 4; ++k) v.v[k] += mult * (f.v[k] * inv * g.v[k] * l.v[k]);
      } else {
#pragma unroll
        for (int k = 0; k < 4; ++k) v.v[k] += mult * (f.v[k] * inv * g.v[k]);
      }
#pragma unroll
      for (int k = 0; k < 4; ++k) sx += v.v[k] * v.v[k];
      Pack4<float>::store(xr + c, v);
      if (next_out != nullptr && next_w == nullptr)
        Pack4<T>::store(next_out + row * width + c, v);
    } else {
      float n = ScalarOps<T>::to_f32(yr[c]) * inv * w[c];
      if (ls != nullptr) n *= ls[c];
      const float v = xr[c] + mult * n;
      xr[c] = v;
      sx += v * v;
      if (next_out != nullptr && next_w == nullptr)
        next_out[row * width + c] = ScalarOps<T>::from_f32(v);
    }
  }
  if (next_w == nullptr) return;
  __syncthreads();
  sx = block_reduce_sum(sx, lds);
  const float inv2 = 1.0f / sqrtf(sx / width + next_eps);
  // every thread re-reads the elements it wrote itself
  for (int c = threadIdx.x * S; c < width; c += blockDim.x * S) {
    if (VEC) {
      F4 v = Pack4<float>::load(xr + c);
      const F4 g = Pack4<float>::load(next_w + c);
#pragma unroll
      for (int k = 0; k < 4; ++k) v.v[k] = v.v[k] * inv2 * (next_offset + g.v[k]);
      Pack4<T>::store(next_out + row * width + c, v);
    } else {
      next_out[row * width + c] =
          ScalarOps<T>::from_f32(xr[c] * inv2 * (next_offset + next_w[c]));
    }
  }
}

template <typename T>
__global__ void softcap_kernel(float* __restrict__ out, const T* __restrict__ in,
                               float cap, long n) {
  const float inv = 1.0f / cap;
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n;
       i += (long)gridDim.x * blockDim.x)
    out[i] = cap * tanhf(ScalarOps<T>::to_f32(in[i]) * inv);
}

// Rotation of dims [offset, offset + 2*half) of every head of x [T, H, D]
// (strided), in place: pair i is dims (i, i + half), or (2i, 2i + 1) when
// `interleaved`.  Angle = float(position) * inv_freq[i]; cos and sin are
// multiplied by `mag`.
template <typename T>
__global__ void rope_partial_kernel(T* __restrict__ x, long st, long sh,
                                    const long* __restrict__ positions,
                                    const float* __restrict__ inv_freq,
                                    int heads, int offset, int half, long n,
                                    int interleaved, float mag) {
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n;
       i += (long)gridDim.x * blockDim.x) {
    const int k = (int)(i % half);
    const long th = i / half;
    const int h = (int)(th % heads);
    const long t = th / heads;
    const float ang = (float)positions[t] * inv_freq[k];
    float s, c;
    sincosf(ang, &s, &c);
    s *= mag;
    c *= mag;
    T* p = x + t * st + h * sh + offset;
    const int ia = interleaved ? 2 * k : k;
    const int ib = interleaved ? 2 * k + 1 : k + half;
    const float u = ScalarOps<T>::to_f32(p[ia]);
    const float v = ScalarOps<T>::to_f32(p[ib]);
    p[ia] = ScalarOps<T>::from_f32(u * c - v * s);
    p[ib] = ScalarOps<T>::from_f32(v * c + u * s);
  }
}

// One workgroup per token: RMS-norm the first `rank` values of the row with a
// plain weight, rotate the first 2*half of the remaining `rot` values (pairs
// and `mag` as in rope_partial), store the row at its slot of the paged cache
// (slot < 0: padding row, skipped).  Input rows are `in_st` elements apart.
template <typename T>
__global__ void latent_kv_write_kernel(const T* __restrict__ dkv,
                                       const float* __restrict__ norm_w,
                                       float eps,
                                       const long* __restrict__ positions,
                                       const float* __restrict__ inv_freq,
                                       int half, T* __restrict__ cache,
                                       const long* __restrict__ slot_mapping,
                                       int rank, int rot, long in_st,
                                       int interleaved, float mag) {
  const long t = blockIdx.x;
  const long slot = slot_mapping[t];
  if (slot < 0) return;
  const int d = rank + rot;
  const T* in = dkv + t * in_st;
  T* out = cache + slot * d;
  float ss = 0.f;
  for (int c = threadIdx.x; c < rank; c += blockDim.x) {
    const float v = ScalarOps<T>::to_f32(in[c]);
    ss += v * v;
  }
  __shared__ float lds[16];
  ss = block_reduce_sum(ss, lds);
  const float inv = 1.0f / sqrtf(ss / rank + eps);
  for (int c = threadIdx.x; c < rank; c += blockDim.x)
    out[c] = ScalarOps<T>::from_f32(ScalarOps<T>::to_f32(in[c]) * inv * norm_w[c]);
  const float pos = (float)positions[t];
  for (int k = threadIdx.x; k < half; k += blockDim.x) {
    float s, c;
    sincosf(pos * inv_freq[k], &s, &c);
    s *= mag;
    c *= mag;
    const int ia = rank + (interleaved ? 2 * k : k);
    const int ib = rank + (interleaved ? 2 * k + 1 : k + half);
    const float u = ScalarOps<T>::to_f32(in[ia]);
    const float v = ScalarOps<T>::to_f32(in[ib]);
    out[ia] = ScalarOps<T>::from_f32(u * c - v * s);
    out[ib] = ScalarOps<T>::from_f32(v * c + u * s);
  }
  for (int k = 2 * half + threadIdx.x; k < rot; k += blockDim.x)
    out[rank + k] = in[rank + k];
}

// ---------------------------------------------------------------------------
// launchers
// ---------------------------------------------------------------------------

template <typename P>
static inline bool al(const P* p, size_t bytes) {
  return p == nullptr || reinterpret_cast<uintptr_t>(p) % bytes == 0;
}

static inline int grid_for(long n, int block) {
  long g = (n + block - 1) / block;
  return (int)(g < 1 ? 1 : (g > 65535 ? 65535 : g));
}

template <typename T>
void launch_gelu_tanh(T* out, const T* x, long x_stride, const T* mul,
                      long mul_stride, int cols, long n, hipStream_t s) {
  if (cols % 4 == 0 && mul_stride % 4 == 0 && x_stride % 4 == 0 &&
      al(out, 4 * sizeof(T)) && al(x, 4 * sizeof(T)) && al(mul, 4 * sizeof(T)))
    gelu_tanh_kernel<T, true><<<grid_for(n / 4, 256), 256, 0, s>>>(
        out, x, x_stride, mul, mul_stride, cols, n / 4);
  else
    gelu_tanh_kernel<T, false><<<grid_for(n, 256), 256, 0, s>>>(
        out, x, x_stride, mul, mul_stride, cols, n);
}
template <typename T>
void launch_embedding_scaled(float* out, const long* ids, const T* table,
                             float scale, int rows, int width, hipStream_t s) {
  embedding_scaled_kernel<T><<<rows, 256, 0, s>>>(out, ids, table, scale, width);
}
template <typename T>
void launch_rms_norm_stream(T* out, const float* x, const float* w, float eps,
                            float offset, int rows, int width, hipStream_t s) {
  if (width % 4 == 0 && al(out, 4 * sizeof(T)) && al(x, 16) && al(w, 16))
    rms_norm_stream_kernel<T, true><<<rows, 256, 0, s>>>(out, x, w, eps, offset, width);
  else
    rms_norm_stream_kernel<T, false><<<rows, 256, 0, s>>>(out, x, w, eps, offset, width);
}
template <typename T>
void launch_stream_add(float* x, const T* a, const T* b, float mult, T* cast,
                       long n, hipStream_t s) {
  if (n % 4 == 0 && al(x, 16) && al(a, 4 * sizeof(T)) && al(b, 4 * sizeof(T)) &&
      al(cast, 4 * sizeof(T)))
    stream_add_kernel<T, true><<<grid_for(n / 4, 256), 256, 0, s>>>(x, a, b, mult, cast, n / 4);
  else
    stream_add_kernel<T, false><<<grid_for(n, 256), 256, 0, s>>>(x, a, b, mult, cast, n);
}
template <typename T>
void launch_stream_add_rms_norm(float* x, const T* y, const float* w, float eps,
                                float mult, int rows, int width, T* next_out,
                                const float* next_w, float next_eps,
                                float next_offset, const float* ls, hipStream_t s) {
  if (width % 4 == 0 && al(x, 16) && al(y, 4 * sizeof(T)) && al(w, 16) &&
      al(next_out, 4 * sizeof(T)) && al(next_w, 16) && al(ls, 16))
    stream_add_rms_norm_kernel<T, true><<<rows, 256, 0, s>>>(
        x, y, w, eps, mult, width, next_out, next_w, next_eps, next_offset, ls);
  else
    stream_add_rms_norm_kernel<T, false><<<rows, 256, 0, s>>>(
        x, y, w, eps, mult, width, next_out, next_w, next_eps, next_offset, ls);
}
template <typename T>
void launch_softcap(float* out, const T* in, float cap, long n, hipStream_t s) {
  softcap_kernel<T><<<grid_for(n, 256), 256, 0, s>>>(out, in, cap, n);
}
template <typename T>
void launch_rope_partial(T* x, long st, long sh, const long* positions,
                         const float* inv_freq, int rows, int heads, int offset,
                         int half, int interleaved, float mag, hipStream_t s) {
  const long n = (long)rows * heads * half;
  rope_partial_kernel<T><<<grid_for(n, 256), 256, 0, s>>>(
      x, st, sh, positions, inv_freq, heads, offset, half, n, interleaved, mag);
}
template <typename T>
void launch_latent_kv_write(const T* dkv, const float* norm_w, float eps,
                            const long* positions, const float* inv_freq,
                            int half, T* cache, const long* slot_mapping,
                            int rows, int rank, int rot, long in_st,
                            int interleaved, float mag, hipStream_t s) {
  latent_kv_write_kernel<T><<<rows, 128, 0, s>>>(
      dkv, norm_w, eps, positions, inv_freq, half, cache, slot_mapping, rank, rot,
      in_st, interleaved, mag);
}

#define INSTANTIATE(T)                                                          \
  template void launch_gelu_tanh<T>(T*, const T*, long, const T*, long, int,    \
                                    long, hipStream_t);                         \
  template void launch_embedding_scaled<T>(float*, const long*, const T*,       \
                                           float, int, int, hipStream_t);       \
  template void launch_rms_norm_stream<T>(T*, const float*, const float*,       \
                                          float, float, int, int, hipStream_t); \
  template void launch_stream_add<T>(float*, const T*, const T*, float, T*,     \
                                     long, hipStream_t);                        \
  template void launch_stream_add_rms_norm<T>(float*, const T*, const float*,   \
                                              float, float, int, int, T*,       \
                                              const float*, float, float,       \
                                              const float*, hipStream_t);       \
  template void launch_softcap<T>(float*, const T*, float, long, hipStream_t);  \
  template void launch_rope_partial<T>(T*, long, long, const long*,             \
                                       const float*, int, int, int, int, int,   \
                                       float, hipStream_t);                     \
  template void launch_latent_kv_write<T>(const T*, const float*, float,        \
                                          const long*, const float*, int, T*,   \
                                          const long*, int, int, int, long,     \
                                          int, float, hipStream_t);
INSTANTIATE(float)
INSTANTIATE(__hip_bfloat16)
