// Torch bindings of the paged grouped-query attention kernels (generic f32 /
// f16 / bf16, bf16 MFMA decode and prefill, fp8 cache variants).  Compiled
// into `_C` and, with module_attn.cpp, into the small `_C_attn` extension for
// models that need nothing else of `_C`.

#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>

#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

template <typename T>
void launch_paged_decode(T*, const T*, const T*, const T*, const int*,
                         const int*, float, int, int, int, int, int, int,
                         hipStream_t);
template <typename T>
void launch_paged_prefill(T*, const T*, const T*, const T*, const int*,
                          const int*, const int*, float, int, int, int, int,
                          int, int, int, hipStream_t);
void launch_paged_prefill_mfma_v2(__hip_bfloat16*, const __hip_bfloat16*,
                                  const __hip_bfloat16*, const __hip_bfloat16*,
                                  const int*, const int*, const int*, float,
                                  int, int, int, int, int, int, int,
                                  hipStream_t);
void launch_paged_prefill_mfma(__hip_bfloat16*, const __hip_bfloat16*,
                               const __hip_bfloat16*, const __hip_bfloat16*,
                               const int*, const int*, const int*, float, int,
                               int, int, int, int, int, int, hipStream_t);
int decode_mfma_num_partitions(int nseq, int kvh, int max_context);
void launch_paged_decode_mfma_fp8(__hip_bfloat16*, float*, float*,
                                  const __hip_bfloat16*, const unsigned char*,
                                  const unsigned char*, const int*,
                                  const int*, float, int, int, int, int, int,
                                  int, int, hipStream_t);
void launch_paged_prefill_mfma_v2_fp8(__hip_bfloat16*, const __hip_bfloat16*,
                                      const unsigned char*,
                                      const unsigned char*, const int*,
                                      const int*, const int*, float, int, int,
                                      int, int, int, int, int, hipStream_t);
void launch_paged_decode_mfma(__hip_bfloat16*, float*, float*,
                              const __hip_bfloat16*, const __hip_bfloat16*,
                              const __hip_bfloat16*, const int*, const int*,
                              float, int, int, int, int, int, int, int,
                              hipStream_t);

void launch_paged_prefill_mfma_v2_ws(__hip_bfloat16*, const __hip_bfloat16*,
                                     const __hip_bfloat16*, const __hip_bfloat16*,
                                     const int*, const int*, const int*, float,
                                     int, int, int, int, int, int, int, int, int,
                                     float, hipStream_t);
void launch_paged_prefill_mfma_v2_chunk(float*, const __hip_bfloat16*,
                                        const __hip_bfloat16*, const __hip_bfloat16*,
                                        const int*, const int*, const int*, float,
                                        int, int, int, int, int, int, int, int,
                                        hipStream_t);
void launch_paged_decode_mfma_chunk(float*, float*, float*, const __hip_bfloat16*,
                                    const __hip_bfloat16*, const __hip_bfloat16*,
                                    const int*, const int*, float, int, int, int,
                                    int, int, int, int, int, int, hipStream_t);
void launch_paged_decode_mfma_ws(__hip_bfloat16*, float*, float*,
                                 const __hip_bfloat16*, const __hip_bfloat16*,
                                 const __hip_bfloat16*, const int*, const int*,
                                 float, int, int, int, int, int, int, int, int,
                                 int, float, hipStream_t);

namespace {

hipStream_t current_stream() {
  return at::hip::getCurrentHIPStream().stream();
}

template <typename T>
T* ptr(torch::Tensor& t) {
  return reinterpret_cast<T*>(t.data_ptr());
}
template <typename T>
const T* cptr(const torch::Tensor& t) {
  return reinterpret_cast<const T*>(t.data_ptr());
}

#define DISPATCH_FLOATING(DTYPE, BODY)                                   \
  switch (DTYPE) {                                                       \
    case at::ScalarType::BFloat16: {                                     \
      using scalar_t = __hip_bfloat16;                                   \
      BODY;                                                              \
      break;                                                             \
    }                                                                    \
    case at::ScalarType::Half: {                                         \
      using scalar_t = __half;                                           \
      BODY;                                                              \
      break;                                                             \
    }                                                                    \
    case at::ScalarType::Float: {                                        \
      using scalar_t = float;                                            \
      BODY;                                                              \
      break;                                                             \
    }                                                                    \
    default:                                                             \
      TORCH_CHECK(false, "unsupported dtype");                           \
  }

void paged_attention_decode(torch::Tensor out, torch::Tensor q,
                            torch::Tensor k_cache, torch::Tensor v_cache,
                            torch::Tensor block_tables, torch::Tensor seq_lens,
                            double scale) {
  const int nseq = q.size(0);
  const int nheads = q.size(1);
  const int head_dim = q.size(2);
  const int kvh = k_cache.size(2);
  const int block_size = k_cache.size(1);
  const int max_blocks = block_tables.size(1);
  TORCH_CHECK(block_tables.scalar_type() == at::ScalarType::Int);
  TORCH_CHECK(seq_lens.scalar_type() == at::ScalarType::Int);
  const int group = nheads / kvh;
  static const bool force_valu = [] {
    const char* e = getenv("VTA_DECODE_VALU");
    return e && e[0] == '1';
  }();
  const bool kv_fp8 = k_cache.scalar_type() == at::ScalarType::Byte;
  if (kv_fp8) {
    TORCH_CHECK(q.scalar_type() == at::ScalarType::BFloat16 &&
                    (head_dim == 64 || head_dim == 128) && group >= 1 &&
                    group <= 8,
                "fp8 KV cache requires the bf16 MFMA decode path");
    const int npart = decode_mfma_num_partitions(nseq, kvh, max_blocks * block_size);
    const int P = npart * 4;
    auto opts = q.options().dtype(at::ScalarType::Float);
    auto part_acc = at::empty({nseq, nheads, P, head_dim}, opts);
    auto part_ml = at::empty({nseq, nheads, P, 2}, opts);
    launch_paged_decode_mfma_fp8(
        reinterpret_cast<__hip_bfloat16*>(out.data_ptr()),
        part_acc.data_ptr<float>(), part_ml.data_ptr<float>(),
        reinterpret_cast<const __hip_bfloat16*>(q.data_ptr()),
        reinterpret_cast<const unsigned char*>(k_cache.data_ptr()),
        reinterpret_cast<const unsigned char*>(v_cache.data_ptr()),
        block_tables.data_ptr<int>(), seq_lens.data_ptr<int>(), (float)scale,
        nseq, nheads, kvh, head_dim, block_size, max_blocks, npart,
        current_stream());
    return;
  }
  if (!force_valu && q.scalar_type() == at::ScalarType::BFloat16 &&
      (head_dim == 64 || head_dim == 128) && group >= 1 && group <= 8 &&
      nheads == kvh * group && nseq > 0) {
    const int npart = decode_mfma_num_partitions(nseq, kvh, max_blocks * block_size);
    const int P = npart * 4;
    auto opts = q.options().dtype(at::ScalarType::Float);
    auto part_acc = at::empty({nseq, nheads, P, head_dim}, opts);
    auto part_ml = at::empty({nseq, nheads, P, 2}, opts);
    launch_paged_decode_mfma(
        reinterpret_cast<__hip_bfloat16*>(out.data_ptr()),
        part_acc.data_ptr<float>(), part_ml.data_ptr<float>(),
        reinterpret_cast<const __hip_bfloat16*>(q.data_ptr()),
        reinterpret_cast<const __hip_bfloat16*>(k_cache.data_ptr()),
        reinterpret_cast<const __hip_bfloat16*>(v_cache.data_ptr()),
        block_tables.data_ptr<int>(), seq_lens.data_ptr<int>(), (float)scale,
        nseq, nheads, kvh, head_dim, block_size, max_blocks, npart,
        current_stream());
    return;
  }
  DISPATCH_FLOATING(q.scalar_type(), {
    launch_paged_decode<scalar_t>(
        ptr<scalar_t>(out), cptr<scalar_t>(q), cptr<scalar_t>(k_cache),
        cptr<scalar_t>(v_cache), block_tables.data_ptr<int>(),
        seq_lens.data_ptr<int>(), (float)scale, nseq, nheads, kvh, head_dim,
        block_size, max_blocks, current_stream());
  });
}

void paged_attention_prefill(torch::Tensor out, torch::Tensor q,
                             torch::Tensor k_cache, torch::Tensor v_cache,
                             torch::Tensor block_tables,
                             torch::Tensor query_start_loc,
                             torch::Tensor seq_lens, double scale,
                             int64_t max_query_len) {
  const int nseq = seq_lens.size(0);
  const int nheads = q.size(1);
  const int head_dim = q.size(2);
  const int kvh = k_cache.size(2);
  const int block_size = k_cache.size(1);
  const int max_blocks = block_tables.size(1);
  static const bool force_valu = [] {
    const char* e = getenv("VTA_PREFILL_VALU");
    return e && e[0] == '1';
  }();
  static const bool force_v1 = [] {
    const char* e = getenv("VTA_PREFILL_V1");
    return e && e[0] == '1';
  }();
  if (k_cache.scalar_type() == at::ScalarType::Byte) {
    TORCH_CHECK(q.scalar_type() == at::ScalarType::BFloat16 && head_dim == 128,
                "fp8 KV cache requires the bf16 v2 prefill path (hd=128)");
    launch_paged_prefill_mfma_v2_fp8(
        reinterpret_cast<__hip_bfloat16*>(out.data_ptr()),
        reinterpret_cast<const __hip_bfloat16*>(q.data_ptr()),
        reinterpret_cast<const unsigned char*>(k_cache.data_ptr()),
        reinterpret_cast<const unsigned char*>(v_cache.data_ptr()),
        block_tables.data_ptr<int>(), query_start_loc.data_ptr<int>(),
        seq_lens.data_ptr<int>(), (float)scale, nseq, nheads, kvh, head_dim,
        block_size, max_blocks, (int)max_query_len, current_stream());
    return;
  }
  if (!force_valu && !force_v1 &&
      q.scalar_type() == at::ScalarType::BFloat16 && head_dim == 128) {
    launch_paged_prefill_mfma_v2(
        reinterpret_cast<__hip_bfloat16*>(out.data_ptr()),
        reinterpret_cast<const __hip_bfloat16*>(q.data_ptr()),
        reinterpret_cast<const __hip_bfloat16*>(k_cache.data_ptr()),
        reinterpret_cast<const __hip_bfloat16*>(v_cache.data_ptr()),
        block_tables.data_ptr<int>(), query_start_loc.data_ptr<int>(),
        seq_lens.data_ptr<int>(), (float)scale, nseq, nheads, kvh, head_dim,
        block_size, max_blocks, (int)max_query_len, current_stream());
    return;
  }
  if (!force_valu && q.scalar_type() == at::ScalarType::BFloat16 &&
      (head_dim == 64 || head_dim == 128)) {
    launch_paged_prefill_mfma(
        reinterpret_cast<__hip_bfloat16*>(out.data_ptr()),
        reinterpret_cast<const __hip_bfloat16*>(q.data_ptr()),
        reinterpret_cast<const __hip_bfloat16*>(k_cache.data_ptr()),
        reinterpret_cast<const __hip_bfloat16*>(v_cache.data_ptr()),
        block_tables.data_ptr<int>(), query_start_loc.data_ptr<int>(),
        seq_lens.data_ptr<int>(), (float)scale, nseq, nheads, kvh, head_dim,
        block_size, max_blocks, (int)max_query_len, current_stream());
    return;
  }
  DISPATCH_FLOATING(q.scalar_type(), {
    launch_paged_prefill<scalar_t>(
        ptr<scalar_t>(out), cptr<scalar_t>(q), cptr<scalar_t>(k_cache),
        cptr<scalar_t>(v_cache), block_tables.data_ptr<int>(),
        query_start_loc.data_ptr<int>(), seq_lens.data_ptr<int>(),
        (float)scale, nseq, nheads, kvh, head_dim, block_size, max_blocks,
        (int)max_query_len, current_stream());
  });
}

// Window + sink variants of the bf16 MFMA kernels: position i sees keys j with
// 0 <= i - j < window (0: all j <= i); has_sink: exp(sink) joins the softmax
// denominator.  Key size = value size = 128 (prompt portions) or 64 / 128
// (single queries), up to 8 query heads per key head.
void check_windowed(const torch::Tensor& out, const torch::Tensor& q,
                    const torch::Tensor& k_cache, const torch::Tensor& v_cache,
                    const torch::Tensor& block_tables, const torch::Tensor& seq_lens,
                    int64_t window) {
  TORCH_CHECK(q.is_cuda() && q.dim() == 3 && q.is_contiguous() && out.is_contiguous() &&
              out.sizes() == q.sizes(), "q / out must be contiguous [rows, heads, dim]");
  TORCH_CHECK(q.scalar_type() == at::ScalarType::BFloat16 &&
              out.scalar_type() == at::ScalarType::BFloat16 &&
              k_cache.scalar_type() == at::ScalarType::BFloat16 &&
              v_cache.scalar_type() == at::ScalarType::BFloat16, "bf16 only");
  TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous() && k_cache.dim() == 4 &&
              k_cache.sizes() == v_cache.sizes() && k_cache.size(3) == q.size(2),
              "cache shape");
  const int nheads = q.size(1), kvh = k_cache.size(2);
  TORCH_CHECK(kvh >= 1 && nheads % kvh == 0 && nheads / kvh <= 8, "heads per key head");
  TORCH_CHECK(block_tables.is_cuda() && block_tables.scalar_type() == at::ScalarType::Int &&
              block_tables.dim() == 2 && block_tables.is_contiguous() &&
              block_tables.size(0) >= seq_lens.numel());
  TORCH_CHECK(seq_lens.is_cuda() && seq_lens.scalar_type() == at::ScalarType::Int &&
              seq_lens.is_contiguous());
  TORCH_CHECK(window >= 0, "window");
}

void windowed_attention_prefill(torch::Tensor out, torch::Tensor q,
                                torch::Tensor k_cache, torch::Tensor v_cache,
                                torch::Tensor block_tables,
                                torch::Tensor query_start_loc,
                                torch::Tensor seq_lens, double scale,
                                int64_t max_query_len, int64_t window,
                                bool has_sink, double sink) {
  check_windowed(out, q, k_cache, v_cache, block_tables, seq_lens, window);
  TORCH_CHECK(q.size(2) == 128, "prompt portions need key size 128");
  const int nseq = seq_lens.numel();
  TORCH_CHECK(query_start_loc.is_cuda() && query_start_loc.is_contiguous() &&
              query_start_loc.scalar_type() == at::ScalarType::Int &&
              query_start_loc.numel() == nseq + 1 && max_query_len >= 1);
  if (q.size(0) == 0 || nseq == 0) return;
  launch_paged_prefill_mfma_v2_ws(
      reinterpret_cast<__hip_bfloat16*>(out.data_ptr()),
      reinterpret_cast<const __hip_bfloat16*>(q.data_ptr()),
      reinterpret_cast<const __hip_bfloat16*>(k_cache.data_ptr()),
      reinterpret_cast<const __hip_bfloat16*>(v_cache.data_ptr()),
      block_tables.data_ptr<int>(), query_start_loc.data_ptr<int>(),
      seq_lens.data_ptr<int>(), (float)scale, nseq, (int)q.size(1),
      (int)k_cache.size(2), 128, (int)k_cache.size(1), (int)block_tables.size(1),
      (int)max_query_len, (int)window, has_sink ? 1 : 0, (float)sink,
      current_stream());
}

void windowed_attention_decode(torch::Tensor out, torch::Tensor q,
                               torch::Tensor k_cache, torch::Tensor v_cache,
                               torch::Tensor block_tables, torch::Tensor seq_lens,
                               double scale, int64_t window, bool has_sink,
                               double sink) {
  check_windowed(out, q, k_cache, v_cache, block_tables, seq_lens, window);
  const int nseq = q.size(0), nheads = q.size(1), head_dim = q.size(2);
  TORCH_CHECK(head_dim == 64 || head_dim == 128, "key size 64 or 128");
  TORCH_CHECK(seq_lens.numel() == nseq, "one query row per sequence expected");
  if (nseq == 0) return;
  const int kvh = k_cache.size(2), block_size = k_cache.size(1);
  const int max_blocks = block_tables.size(1);
  // shape-pure split count; a window bounds the keys a query reads
  int span = max_blocks * block_size;
  if (window > 0 && window + 32 < span) span = (int)window + 32;
  const int npart = decode_mfma_num_partitions(nseq, kvh, span);
  const int P = npart * 4;
  auto opts = q.options().dtype(at::ScalarType::Float);
  auto part_acc = at::empty({nseq, nheads, P, head_dim}, opts);
  auto part_ml = at::empty({nseq, nheads, P, 2}, opts);
  launch_paged_decode_mfma_ws(
      reinterpret_cast<__hip_bfloat16*>(out.data_ptr()), part_acc.data_ptr<float>(),
      part_ml.data_ptr<float>(), reinterpret_cast<const __hip_bfloat16*>(q.data_ptr()),
      reinterpret_cast<const __hip_bfloat16*>(k_cache.data_ptr()),
      reinterpret_cast<const __hip_bfloat16*>(v_cache.data_ptr()),
      block_tables.data_ptr<int>(), seq_lens.data_ptr<int>(), (float)scale, nseq,
      nheads, kvh, head_dim, block_size, max_blocks, npart, (int)window,
      has_sink ? 1 : 0, (float)sink, current_stream());
}

// Chunk variants of the bf16 MFMA kernels: position i sees keys j <= i with
// floor(j / chunk) = floor(i / chunk) (0: all j <= i); the value cache may hold
// fewer heads than the key cache (key head g reads value head g mod Gv); the
// output is f32.  Sizes as for the window variants.
void check_chunked(const torch::Tensor& out, const torch::Tensor& q,
                   const torch::Tensor& k_cache, const torch::Tensor& v_cache,
                   const torch::Tensor& block_tables, const torch::Tensor& seq_lens,
                   int64_t chunk) {
  TORCH_CHECK(q.is_cuda() && q.dim() == 3 && q.is_contiguous() && out.is_cuda() &&
              out.is_contiguous() && out.sizes() == q.sizes(),
              "q / out must be contiguous [rows, heads, dim]");
  TORCH_CHECK(q.scalar_type() == at::ScalarType::BFloat16 &&
              out.scalar_type() == at::ScalarType::Float &&
              k_cache.scalar_type() == at::ScalarType::BFloat16 &&
              v_cache.scalar_type() == at::ScalarType::BFloat16, "bf16 in, f32 out");
  TORCH_CHECK(k_cache.is_cuda() && v_cache.is_cuda() && k_cache.is_contiguous() &&
              v_cache.is_contiguous() && k_cache.dim() == 4 && v_cache.dim() == 4 &&
              k_cache.size(0) == v_cache.size(0) && k_cache.size(1) == v_cache.size(1) &&
              k_cache.size(3) == q.size(2) && v_cache.size(3) == q.size(2),
              "cache shape");
  const int nheads = q.size(1), kvh = k_cache.size(2), vh = v_cache.size(2);
  TORCH_CHECK(kvh >= 1 && nheads % kvh == 0 && nheads / kvh <= 8, "heads per key head");
  TORCH_CHECK(vh >= 1 && kvh % vh == 0, "key heads per value head");
  TORCH_CHECK(block_tables.is_cuda() && block_tables.scalar_type() == at::ScalarType::Int &&
              block_tables.dim() == 2 && block_tables.is_contiguous() &&
              block_tables.size(0) >= seq_lens.numel());
  TORCH_CHECK(seq_lens.is_cuda() && seq_lens.scalar_type() == at::ScalarType::Int &&
              seq_lens.is_contiguous());
  TORCH_CHECK(chunk >= 0, "chunk");
}

void chunk_attention_prefill(torch::Tensor out, torch::Tensor q, torch::Tensor k_cache,
                             torch::Tensor v_cache, torch::Tensor block_tables,
                             torch::Tensor query_start_loc, torch::Tensor seq_lens,
                             double scale, int64_t max_query_len, int64_t chunk) {
  check_chunked(out, q, k_cache, v_cache, block_tables, seq_lens, chunk);
  TORCH_CHECK(q.size(2) == 128, "prompt portions need key size 128");
  const int nseq = seq_lens.numel();
  TORCH_CHECK(query_start_loc.is_cuda() && query_start_loc.is_contiguous() &&
              query_start_loc.scalar_type() == at::ScalarType::Int &&
              query_start_loc.numel() == nseq + 1 && max_query_len >= 1);
  if (q.size(0) == 0 || nseq == 0) return;
  launch_paged_prefill_mfma_v2_chunk(
      out.data_ptr<float>(), reinterpret_cast<const __hip_bfloat16*>(q.data_ptr()),
      reinterpret_cast<const __hip_bfloat16*>(k_cache.data_ptr()),
      reinterpret_cast<const __hip_bfloat16*>(v_cache.data_ptr()),
      block_tables.data_ptr<int>(), query_start_loc.data_ptr<int>(),
      seq_lens.data_ptr<int>(), (float)scale, nseq, (int)q.size(1),
      (int)k_cache.size(2), (int)v_cache.size(2), (int)k_cache.size(1),
      (int)block_tables.size(1), (int)max_query_len, (int)chunk, current_stream());
}

void chunk_attention_decode(torch::Tensor out, torch::Tensor q, torch::Tensor k_cache,
                            torch::Tensor v_cache, torch::Tensor block_tables,
                            torch::Tensor seq_lens, double scale, int64_t chunk) {
  check_chunked(out, q, k_cache, v_cache, block_tables, seq_lens, chunk);
  const int nseq = q.size(0), nheads = q.size(1), head_dim = q.size(2);
  TORCH_CHECK(head_dim == 64 || head_dim == 128, "key size 64 or 128");
  TORCH_CHECK(seq_lens.numel() == nseq, "one query row per sequence expected");
  if (nseq == 0) return;
  const int kvh = k_cache.size(2), block_size = k_cache.size(1);
  const int max_blocks = block_tables.size(1);
  // shape-pure split count; a chunk bounds the keys a query reads
  int span = max_blocks * block_size;
  if (chunk > 0 && chunk + 32 < span) span = (int)chunk + 32;
  const int npart = decode_mfma_num_partitions(nseq, kvh, span);
  const int P = npart * 4;
  auto opts = q.options().dtype(at::ScalarType::Float);
  auto part_acc = at::empty({nseq, nheads, P, head_dim}, opts);
  auto part_ml = at::empty({nseq, nheads, P, 2}, opts);
  launch_paged_decode_mfma_chunk(
      out.data_ptr<float>(), part_acc.data_ptr<float>(), part_ml.data_ptr<float>(),
      reinterpret_cast<const __hip_bfloat16*>(q.data_ptr()),
      reinterpret_cast<const __hip_bfloat16*>(k_cache.data_ptr()),
      reinterpret_cast<const __hip_bfloat16*>(v_cache.data_ptr()),
      block_tables.data_ptr<int>(), seq_lens.data_ptr<int>(), (float)scale, nseq,
      nheads, kvh, (int)v_cache.size(2), head_dim, block_size, max_blocks, npart,
      (int)chunk, current_stream());
}

}  // namespace

void register_attention_ops(pybind11::module& m) {
  m.def("chunk_attention_prefill", &chunk_attention_prefill,
        "paged chunk-masked prefill attention, f32 out (CDNA4)");
  m.def("chunk_attention_decode", &chunk_attention_decode,
        "paged chunk-masked decode attention, f32 out (CDNA4)");
  m.def("windowed_attention_prefill", &windowed_attention_prefill,
        "paged windowed prefill attention with a softmax sink (CDNA4)");
  m.def("windowed_attention_decode", &windowed_attention_decode,
        "paged windowed decode attention with a softmax sink (CDNA4)");
  m.def("paged_attention_decode", &paged_attention_decode,
        "paged decode attention (CDNA4)");
  m.def("paged_attention_prefill", &paged_attention_prefill,
        "paged causal prefill attention (CDNA4)");
}
