// Torch bindings of the `_C_lat` extension: windowed latent attention with
// sinks (general and MFMA kernels).

#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>

#include <hip/hip_bf16.h>

template <typename T>
void launch_latent_attention(T*, long, long, const T*, long, long, const T*,
                             long, long, const T*, const int*, int, const int*,
                             const int*, int, const float*, float, int, int,
                             int, int, int, int, hipStream_t);
bool latent_prefill_mfma_usable(int rank, int rot, int block_size);
void launch_latent_attn_mfma(__hip_bfloat16*, long, long,
                             const __hip_bfloat16*, long, long,
                             const __hip_bfloat16*, long, long,
                             const __hip_bfloat16*, const int*, int, const int*,
                             const int*, int, const float*, float, int, int,
                             int, int, int, int, int, int, float*, float*,
                             hipStream_t);
int latent_decode_num_splits(int nseq, int heads, int max_keys);

namespace {

hipStream_t stream() { return at::hip::getCurrentHIPStream().stream(); }

template <typename T>
T* ptr(const torch::Tensor& t) {
  return reinterpret_cast<T*>(t.data_ptr());
}

#define DISPATCH_F32_BF16(DTYPE, BODY)                                  \
  switch (DTYPE) {                                                      \
    case at::ScalarType::BFloat16: {                                    \
      using scalar_t = __hip_bfloat16;                                  \
      BODY;                                                             \
      break;                                                            \
    }                                                                   \
    case at::ScalarType::Float: {                                       \
      using scalar_t = float;                                           \
      BODY;                                                             \
      break;                                                            \
    }                                                                   \
    default:                                                            \
      TORCH_CHECK(false, "this op takes float32 or bfloat16 tensors");  \
  }

void check_f32(const torch::Tensor& t, const char* what) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::ScalarType::Float &&
                  t.is_contiguous(), what, " must be a contiguous f32 GPU tensor");
}
void check_i32(const torch::Tensor& t, const char* what) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::ScalarType::Int &&
                  t.is_contiguous(), what, " must be a contiguous int32 GPU tensor");
}
void check_i64(const torch::Tensor& t, const char* what) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::ScalarType::Long &&
                  t.is_contiguous(), what, " must be a contiguous int64 GPU tensor");
}

void latent_attention_common(torch::Tensor& out, torch::Tensor& q_lat,
                             torch::Tensor& q_rot, torch::Tensor& cache,
                             torch::Tensor& block_tables, const int* qsl,
                             torch::Tensor& seq_lens, double scale,
                             int64_t window,
                             c10::optional<torch::Tensor>& sinks,
                             int max_q, bool allow_mfma, bool two_term) {
  TORCH_CHECK(q_lat.is_cuda() && q_lat.dim() == 3 && q_rot.dim() == 3 &&
              out.dim() == 3);
  TORCH_CHECK(q_lat.stride(2) == 1 && q_rot.stride(2) == 1 && out.stride(2) == 1);
  const int rows = q_lat.size(0), heads = q_lat.size(1), rank = q_lat.size(2);
  const int rot = q_rot.size(2);
  TORCH_CHECK(q_rot.size(0) == rows && q_rot.size(1) == heads &&
              out.size(0) == rows && out.size(1) == heads && out.size(2) == rank);
  TORCH_CHECK(cache.is_contiguous() && cache.dim() == 3 &&
              cache.size(2) == rank + rot, "latent cache row size");
  TORCH_CHECK(cache.scalar_type() == q_lat.scalar_type() &&
              q_rot.scalar_type() == q_lat.scalar_type() &&
              out.scalar_type() == q_lat.scalar_type());
  TORCH_CHECK(rank <= 1024, "latent rank above 1024 is not supported");
  check_i32(seq_lens, "seq_lens");
  TORCH_CHECK(block_tables.is_cuda() &&
              block_tables.scalar_type() == at::ScalarType::Int &&
              block_tables.dim() == 2 && block_tables.stride(1) == 1);
  const int nseq = seq_lens.numel();
  TORCH_CHECK(block_tables.size(0) >= nseq);
  TORCH_CHECK(qsl != nullptr || rows == nseq);
  const float* sk = nullptr;
  if (sinks.has_value()) {
    check_f32(sinks.value(), "sinks");
    TORCH_CHECK(sinks.value().numel() == heads);
    sk = ptr<float>(sinks.value());
  }
  const int block_size = cache.size(1);
  auto vec_ok = [](const torch::Tensor& t, int elems) {
    return t.stride(0) % elems == 0 && t.stride(1) % elems == 0 &&
           reinterpret_cast<uintptr_t>(t.data_ptr()) % (2 * elems) == 0;
  };
  if (allow_mfma && q_lat.scalar_type() == at::ScalarType::BFloat16 &&
      latent_prefill_mfma_usable(rank, rot, block_size) && vec_ok(q_lat, 8) &&
      vec_ok(q_rot, 8) && vec_ok(out, 4)) {
    using bf = __hip_bfloat16;
    // single-query steps: slice the keys over workgroups (shape-pure count)
    int nsplit = 1;
    torch::Tensor part_acc, part_ml;
    if (qsl == nullptr) {
      const int max_keys = window > 0
          ? (int)window : (int)(block_tables.size(1) * block_size);
      nsplit = latent_decode_num_splits(nseq, heads, max_keys);
      if (nsplit > 1) {
        auto opt = torch::TensorOptions().dtype(torch::kFloat32).device(out.device());
        part_acc = torch::empty({(long)nseq * nsplit * heads * rank}, opt);
        part_ml = torch::empty({(long)nseq * nsplit * heads * 2}, opt);
      }
    }
    launch_latent_attn_mfma(
        ptr<bf>(out), out.stride(0), out.stride(1), ptr<bf>(q_lat),
        q_lat.stride(0), q_lat.stride(1), ptr<bf>(q_rot), q_rot.stride(0),
        q_rot.stride(1), ptr<bf>(cache), ptr<int>(block_tables),
        (int)block_tables.stride(0), qsl, ptr<int>(seq_lens), nseq, sk,
        (float)scale, (int)window, max_q, heads, rank, rot, block_size, nsplit,
        two_term ? 1 : 0, nsplit > 1 ? ptr<float>(part_acc) : nullptr,
        nsplit > 1 ? ptr<float>(part_ml) : nullptr, stream());
    return;
  }
  DISPATCH_F32_BF16(q_lat.scalar_type(), {
    launch_latent_attention<scalar_t>(
        ptr<scalar_t>(out), out.stride(0), out.stride(1), ptr<scalar_t>(q_lat),
        q_lat.stride(0), q_lat.stride(1), ptr<scalar_t>(q_rot), q_rot.stride(0),
        q_rot.stride(1), ptr<scalar_t>(cache), ptr<int>(block_tables),
        (int)block_tables.stride(0), qsl, ptr<int>(seq_lens), nseq, sk,
        (float)scale, (int)window, rows, heads, rank, rot, block_size, stream());
  });
}

void latent_attention_prefill(torch::Tensor out, torch::Tensor q_lat,
                              torch::Tensor q_rot, torch::Tensor cache,
                              torch::Tensor block_tables, torch::Tensor qsl,
                              torch::Tensor seq_lens, double scale,
                              int64_t window, c10::optional<torch::Tensor> sinks,
                              int64_t max_query_len, bool generic,
                              bool two_term) {
  check_i32(qsl, "query_start_loc");
  TORCH_CHECK(qsl.numel() == seq_lens.numel() + 1);
  TORCH_CHECK(max_query_len >= 1, "max_query_len");
  latent_attention_common(out, q_lat, q_rot, cache, block_tables, ptr<int>(qsl),
                          seq_lens, scale, window, sinks, (int)max_query_len,
                          !generic, two_term);
}

void latent_attention_decode(torch::Tensor out, torch::Tensor q_lat,
                             torch::Tensor q_rot, torch::Tensor cache,
                             torch::Tensor block_tables, torch::Tensor seq_lens,
                             double scale, int64_t window,
                             c10::optional<torch::Tensor> sinks, bool generic,
                             bool two_term) {
  latent_attention_common(out, q_lat, q_rot, cache, block_tables, nullptr,
                          seq_lens, scale, window, sinks, 1, !generic, two_term);
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("latent_attention_prefill", &latent_attention_prefill);
  m.def("latent_attention_decode", &latent_attention_decode);
}
