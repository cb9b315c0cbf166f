// Causal grouped-query softmax attention over a paged K/V cache for any
// query/key size, any value size (it need not equal the key size), f32 or
// bf16 storage; scores, softmax and accumulation in f32.
//
//   k_cache [blocks, block, G, dim]     v_cache [blocks, block, G, vdim]
//   q [rows, H, dim]  ->  out [rows, H, vdim]
//
// Query head h reads key/value head h / (H / G).  A query at position i sees
// keys j with 0 <= i - j < window (window 0: every j <= i); with a sink the
// softmax denominator also holds exp(sink), a key without a value; with a
// chunk size c it sees only keys of its own chunk, floor(j / c) = floor(i / c),
// chunks counted from position 0.  The value cache may hold fewer heads Gv
// than the key cache: key head g reads value head g mod Gv.  The output type
// may be f32 beside a 16-bit cache.  One workgroup per (query row, head).  Per tile of 256 keys:
//   phase 1  thread j scores key j (q, already multiplied by the score scale,
//            broadcast from LDS; the key row read with 16-byte loads), block
//            max / sum give the online-softmax step
//   phase 2  threads regroup as (key group g, value dim k): group g sums
//            p_j * v_j[k] over the keys j = g mod G of the tile, loads of
//            v_j[k] coalesced over k
// The groups are summed through LDS at the end.  Decode (one query per
// sequence, qsl == nullptr) and prompt portions (rows located through
// query_start_loc) share the kernel.  This is the path for f32 and for shapes
// the MFMA kernels do not take.

#include "common.h"

namespace {

constexpr int PA_THREADS = 256;
constexpr int PA_MAX_DPT = 4;   // value dims per thread: vdim <= 1024

DEVINLINE float pa_reduce_max(float x, float* scratch) {
  const int lane = threadIdx.x & (WAVE_SIZE - 1);
  const int wave = threadIdx.x / WAVE_SIZE;
  x = wave_reduce_max(x);
  __syncthreads();
  if (lane == 0) scratch[wave] = x;
  __syncthreads();
  float m = -INFINITY;
  for (int i = 0; i < PA_THREADS / WAVE_SIZE; ++i) m = fmaxf(m, scratch[i]);
  __syncthreads();
  return m;
}

DEVINLINE float pa_reduce_sum(float x, float* scratch) {
  const int lane = threadIdx.x & (WAVE_SIZE - 1);
  const int wave = threadIdx.x / WAVE_SIZE;
  x = wave_reduce_sum(x);
  __syncthreads();
  if (lane == 0) scratch[wave] = x;
  __syncthreads();
  float s = 0.f;
  for (int i = 0; i < PA_THREADS / WAVE_SIZE; ++i) s += scratch[i];
  __syncthreads();
  return s;
}

template <typename T, typename O>
__global__ __launch_bounds__(PA_THREADS) void paged_attention_any_kernel(
    O* __restrict__ out, long o_st, const T* __restrict__ q, long q_st,
    const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_tables, int bt_stride,
    const int* __restrict__ qsl, const int* __restrict__ seq_lens, int nseq,
    float scale, int heads, int kv_heads, int dim, int vdim, int block_size,
    int vp /* pow2 >= min(vdim, 256) */, int vec_ok, int window, int has_sink,
    float sink, int chunk, int v_heads) {
  extern __shared__ float smem[];
  float* q_s = smem;                               // [dim]
  float* p_s = q_s + ((dim + 1) & ~1);             // [256]
  long* tok_s = reinterpret_cast<long*>(p_s + PA_THREADS);    // [256] cache token index
  float* red = reinterpret_cast<float*>(tok_s + PA_THREADS);  // [16]
  float* acc_s = red + 16;                         // [256]

  const int row = blockIdx.x;
  const int h = blockIdx.y;
  const int g_kv = h / (heads / kv_heads);
  const int tid = threadIdx.x;

  int seq, ctx;
  if (qsl != nullptr) {
    int lo = 0, hi = nseq;
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (qsl[mid] <= row) lo = mid; else hi = mid;
    }
    seq = lo;
    const int n = qsl[seq + 1] - qsl[seq];
    ctx = seq_lens[seq] - n + (row - qsl[seq]) + 1;
  } else {
    seq = row;
    ctx = seq_lens[row];
  }
  const int g_v = g_kv % v_heads;
  O* orow = out + row * o_st + (long)h * vdim;
  if (ctx <= 0) {
    for (int k = tid; k < vdim; k += PA_THREADS) orow[k] = ScalarOps<O>::from_f32(0.f);
    return;
  }
  const T* qr = q + row * q_st + (long)h * dim;
  for (int k = tid; k < dim; k += PA_THREADS) q_s[k] = ScalarOps<T>::to_f32(qr[k]) * scale;
  __syncthreads();

  constexpr int V = Vec16<T>::kElems;
  const int* bt = block_tables + (long)seq * bt_stride;
  const long k_tok = (long)kv_heads * dim;     // elements per cached token
  const long v_tok = (long)v_heads * vdim;

  const int groups = PA_THREADS / vp;          // >= 1
  const int g = tid / vp;
  const int k0 = tid - g * vp;
  float acc[PA_MAX_DPT];
#pragma unroll
  for (int i = 0; i < PA_MAX_DPT; ++i) acc[i] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  int first = (window > 0 && ctx > window) ? ctx - window : 0;
  if (chunk > 0) first = max(first, ((ctx - 1) / chunk) * chunk);
  for (int base = first; base < ctx; base += PA_THREADS) {
    const int j = base + tid;
    float s = -INFINITY;
    if (j < ctx) {
      const long tok = (long)bt[j / block_size] * block_size + (j % block_size);
      tok_s[tid] = tok;
      const T* kr = k_cache + tok * k_tok + (long)g_kv * dim;
      float a = 0.f;
      if (vec_ok) {
        for (int k = 0; k < dim; k += V) {
          const Vec16<T> v = load16(kr + k);
#pragma unroll
          for (int u = 0; u < V; ++u) a += q_s[k + u] * ScalarOps<T>::to_f32(v.data[u]);
        }
      } else {
        for (int k = 0; k < dim; ++k) a += q_s[k] * ScalarOps<T>::to_f32(kr[k]);
      }
      s = a;
    }
    const float m_tile = pa_reduce_max(s, red);
    const float m_new = fmaxf(m_run, m_tile);
    const float alpha = (m_run == -INFINITY) ? 0.f : expf(m_run - m_new);
    const float p = (j < ctx) ? expf(s - m_new) : 0.f;
    p_s[tid] = p;
    const float l_tile = pa_reduce_sum(p, red);   // its barriers also publish p_s / tok_s
    l_run = l_run * alpha + l_tile;
    m_run = m_new;
    const int nk = min(PA_THREADS, ctx - base);
#pragma unroll
    for (int i = 0; i < PA_MAX_DPT; ++i) acc[i] *= alpha;
    for (int jj = g; jj < nk; jj += groups) {
      const float pj = p_s[jj];
      const T* vr = v_cache + tok_s[jj] * v_tok + (long)g_v * vdim;
#pragma unroll
      for (int i = 0; i < PA_MAX_DPT; ++i) {
        const int k = k0 + i * vp;
        if (k < vdim) acc[i] += pj * ScalarOps<T>::to_f32(vr[k]);
      }
    }
    __syncthreads();   // p_s / tok_s are rewritten by the next tile
  }

  float inv = 1.0f / l_run;
  if (has_sink) {
    const float m_fin = fmaxf(m_run, sink);
    const float rescale = expf(m_run - m_fin);
    inv = rescale / (l_run * rescale + expf(sink - m_fin));
  }
  if (groups > 1) {
    // vdim <= vp <= 128 here: one dim per thread, sum the groups through LDS
    acc_s[tid] = acc[0];
    __syncthreads();
    if (g == 0 && k0 < vdim) {
      float a = 0.f;
      for (int gg = 0; gg < groups; ++gg) a += acc_s[gg * vp + k0];
      orow[k0] = ScalarOps<O>::from_f32(a * inv);
    }
  } else {
#pragma unroll
    for (int i = 0; i < PA_MAX_DPT; ++i) {
      const int k = k0 + i * vp;
      if (k < vdim) orow[k] = ScalarOps<O>::from_f32(acc[i] * inv);
    }
  }
}

}  // namespace

template <typename T, typename O>
static void launch_any(O* out, long o_st, const T* q, long q_st, const T* k_cache,
                       const T* v_cache, const int* block_tables, int bt_stride,
                       const int* qsl, const int* seq_lens, int nseq, float scale,
                       int rows, int heads, int kv_heads, int dim, int vdim,
                       int block_size, int vec_ok, int window, int has_sink,
                       float sink, int chunk, int v_heads, hipStream_t stream) {
  int vp = 1;
  while (vp < vdim && vp < PA_THREADS) vp <<= 1;
  const size_t smem = sizeof(float) * (((dim + 1) & ~1) + PA_THREADS + 16 + PA_THREADS) +
                      sizeof(long) * PA_THREADS;
  dim3 grid(rows, heads);
  paged_attention_any_kernel<T, O><<<grid, PA_THREADS, smem, stream>>>(
      out, o_st, q, q_st, k_cache, v_cache, block_tables, bt_stride, qsl,
      seq_lens, nseq, scale, heads, kv_heads, dim, vdim, block_size, vp, vec_ok,
      window, has_sink, sink, chunk, v_heads);
}

template <typename T>
void launch_paged_attention_any(T* out, long o_st, const T* q, long q_st,
                                const T* k_cache, const T* v_cache,
                                const int* block_tables, int bt_stride,
                                const int* qsl, const int* seq_lens, int nseq,
                                float scale, int rows, int heads, int kv_heads,
                                int dim, int vdim, int block_size, int vec_ok,
                                int window, int has_sink, float sink,
                                hipStream_t stream) {
  launch_any<T, T>(out, o_st, q, q_st, k_cache, v_cache, block_tables, bt_stride, qsl,
                   seq_lens, nseq, scale, rows, heads, kv_heads, dim, vdim,
                   block_size, vec_ok, window, has_sink, sink, 0, kv_heads, stream);
}

// chunk-masked variant with f32 output and a value cache of v_heads heads
template <typename T>
void launch_chunk_attention(float* out, long o_st, const T* q, long q_st,
                            const T* k_cache, const T* v_cache,
                            const int* block_tables, int bt_stride, const int* qsl,
                            const int* seq_lens, int nseq, float scale, int rows,
                            int heads, int kv_heads, int v_heads, int dim, int vdim,
                            int block_size, int vec_ok, int chunk,
                            hipStream_t stream) {
  launch_any<T, float>(out, o_st, q, q_st, k_cache, v_cache, block_tables, bt_stride,
                       qsl, seq_lens, nseq, scale, rows, heads, kv_heads, dim, vdim,
                       block_size, vec_ok, 0, 0, 0.f, chunk, v_heads, stream);
}

template void launch_paged_attention_any<float>(
    float*, long, const float*, long, const float*, const float*, const int*, int,
    const int*, const int*, int, float, int, int, int, int, int, int, int, int,
    int, float, hipStream_t);
template void launch_paged_attention_any<__hip_bfloat16>(
    __hip_bfloat16*, long, const __hip_bfloat16*, long, const __hip_bfloat16*,
    const __hip_bfloat16*, const int*, int, const int*, const int*, int, float,
    int, int, int, int, int, int, int, int, int, float, hipStream_t);
template void launch_chunk_attention<float>(
    float*, long, const float*, long, const float*, const float*, const int*, int,
    const int*, const int*, int, float, int, int, int, int, int, int, int, int,
    int, hipStream_t);
template void launch_chunk_attention<__hip_bfloat16>(
    float*, long, const __hip_bfloat16*, long, const __hip_bfloat16*,
    const __hip_bfloat16*, const int*, int, const int*, const int*, int, float,
    int, int, int, int, int, int, int, int, int, hipStream_t);
