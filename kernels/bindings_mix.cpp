// Torch bindings (part of `_C_seq`): token shift with a carried row, query/key
// norm + rotation + cache write, chunk-masked attention with f32 output, the
// differential combination, RMS norm in groups, the HGRN2 recurrence and the
// gated activation with a weight per (row, expert).  Every shape the kernels
// assume is checked here, on the host, before a launch.

#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>

#include <hip/hip_bf16.h>

template <typename T>
void launch_token_shift_state(T*, const float*, const float*, float*, const int*,
                              const int*, const int*, int, int, int, hipStream_t);
template <typename T>
void launch_qk_norm_rope_cache_write(T*, const T*, long, const T*, long, const T*,
                                     long, const float*, const float*, float,
                                     const long*, const float*, int, T*, T*,
                                     const long*, int, int, int, int, int, int,
                                     hipStream_t);
template <typename T>
void launch_diff_combine(T*, const float*, float, float, float, const T*, long, int,
                         int, int, hipStream_t);
template <typename T, typename I>
void launch_group_rms_norm(T*, const I*, const float*, float, long, int, int,
                           hipStream_t);
template <typename T>
void launch_silu_mul_scaled(T*, const T*, const float*, long, int, int, hipStream_t);
template <typename T>
void launch_chunk_attention(float*, long, const T*, long, const T*, const T*,
                            const int*, int, const int*, const int*, int, float,
                            int, int, int, int, int, int, int, int, int,
                            hipStream_t);
template <typename T>
void launch_hgrn2_scan(float*, const T*, long, const T*, long, const T*, long,
                       const float*, const float*, float*, const int*, const int*,
                       const int*, int, int, int, int, int, float*, int,
                       hipStream_t);

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
bool aligned16(const torch::Tensor& t) {
  return reinterpret_cast<uintptr_t>(t.data_ptr()) % 16 == 0;
}
bool is_f32_or_bf16(const torch::Tensor& t) {
  return t.scalar_type() == at::ScalarType::Float ||
         t.scalar_type() == at::ScalarType::BFloat16;
}

int check_seqs(const torch::Tensor& loc, const torch::Tensor& seq_lens,
               const torch::Tensor& slots) {
  check_i32(loc, "seq_start_loc");
  check_i32(seq_lens, "seq_lens");
  check_i32(slots, "state_slots");
  const int nseq = seq_lens.numel();
  TORCH_CHECK(loc.numel() == nseq + 1 && slots.numel() == nseq,
              "seq_start_loc / seq_lens / state_slots do not fit each other");
  return nseq;
}

// heads of one row laid out [heads, size] with unit stride, rows strided
void check_heads_view(const torch::Tensor& t, const char* what) {
  TORCH_CHECK(t.is_cuda() && t.dim() == 3 && t.stride(2) == 1 &&
                  t.stride(1) == t.size(2), what, " must be [rows, heads, size] rows");
}

void token_shift_state(torch::Tensor out, torch::Tensor x, torch::Tensor weight,
                       torch::Tensor state, torch::Tensor loc, torch::Tensor seq_lens,
                       torch::Tensor slots) {
  const int nseq = check_seqs(loc, seq_lens, slots);
  check_f32(x, "x");
  check_f32(weight, "weight");
  check_f32(state, "state");
  TORCH_CHECK(x.dim() == 2 && out.is_cuda() && out.is_contiguous() &&
              out.sizes() == x.sizes() && is_f32_or_bf16(out));
  const int rows = x.size(0), width = x.size(1);
  TORCH_CHECK(weight.numel() == width && state.dim() == 2 && state.size(1) == width);
  if (rows == 0 || nseq == 0) return;
  DISPATCH_F32_BF16(out.scalar_type(), {
    launch_token_shift_state<scalar_t>(ptr<scalar_t>(out), ptr<float>(x),
                                       ptr<float>(weight), ptr<float>(state),
                                       ptr<int>(loc), ptr<int>(seq_lens),
                                       ptr<int>(slots), nseq, rows, width, stream());
  });
}

void qk_norm_rope_cache_write(torch::Tensor q_out, torch::Tensor q, torch::Tensor k,
                              torch::Tensor v, torch::Tensor q_weight,
                              torch::Tensor k_weight, double eps,
                              torch::Tensor positions, torch::Tensor inv_freq,
                              int64_t rot_dims, torch::Tensor k_cache,
                              torch::Tensor v_cache, torch::Tensor slot_mapping) {
  check_heads_view(q, "q");
  check_heads_view(k, "k");
  check_heads_view(v, "v");
  check_f32(q_weight, "q_weight");
  check_f32(k_weight, "k_weight");
  check_f32(inv_freq, "inv_freq");
  check_i64(positions, "positions");
  check_i64(slot_mapping, "slot_mapping");
  const int tokens = q.size(0), heads = q.size(1), dim = q.size(2);
  const int kv_heads = k.size(1), v_heads = v.size(1), vdim = v.size(2);
  const auto dt = q.scalar_type();
  TORCH_CHECK(k.size(0) == tokens && v.size(0) == tokens && k.size(2) == dim);
  TORCH_CHECK(k.scalar_type() == dt && v.scalar_type() == dt &&
              q_out.scalar_type() == dt && k_cache.scalar_type() == dt &&
              v_cache.scalar_type() == dt);
  TORCH_CHECK(q_out.is_cuda() && q_out.is_contiguous() && q_out.numel() == q.numel());
  TORCH_CHECK(q_weight.numel() == dim && k_weight.numel() == dim);
  TORCH_CHECK(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= dim &&
              inv_freq.numel() >= rot_dims / 2, "rotated dims");
  TORCH_CHECK(positions.numel() == tokens && slot_mapping.numel() == tokens);
  TORCH_CHECK(k_cache.is_cuda() && k_cache.is_contiguous() && k_cache.dim() == 4 &&
              k_cache.size(2) == kv_heads && k_cache.size(3) == dim &&
              v_cache.is_cuda() && v_cache.is_contiguous() && v_cache.dim() == 4 &&
              v_cache.size(2) == v_heads && v_cache.size(3) == vdim &&
              v_cache.size(0) == k_cache.size(0) && v_cache.size(1) == k_cache.size(1),
              "cache shape");
  TORCH_CHECK(dim <= 4096, "head size");
  if (tokens == 0) return;
  DISPATCH_F32_BF16(dt, {
    launch_qk_norm_rope_cache_write<scalar_t>(
        ptr<scalar_t>(q_out), ptr<scalar_t>(q), (long)q.stride(0), ptr<scalar_t>(k),
        (long)k.stride(0), ptr<scalar_t>(v), (long)v.stride(0), ptr<float>(q_weight),
        ptr<float>(k_weight), (float)eps, ptr<long>(positions), ptr<float>(inv_freq),
        (int)rot_dims, ptr<scalar_t>(k_cache), ptr<scalar_t>(v_cache),
        ptr<long>(slot_mapping), tokens, heads, kv_heads, v_heads, dim, vdim, stream());
  });
}

void chunk_attention(torch::Tensor out, torch::Tensor q, torch::Tensor k_cache,
                     torch::Tensor v_cache, torch::Tensor block_tables,
                     c10::optional<torch::Tensor> query_start_loc,
                     torch::Tensor seq_lens, double scale, int64_t max_query_len,
                     int64_t chunk) {
  TORCH_CHECK(q.is_cuda() && q.dim() == 3 && out.is_cuda() && out.dim() == 3 &&
              out.scalar_type() == at::ScalarType::Float);
  TORCH_CHECK(chunk >= 0, "chunk");
  const int rows = q.size(0), heads = q.size(1), dim = q.size(2);
  TORCH_CHECK(k_cache.is_cuda() && v_cache.is_cuda() && k_cache.is_contiguous() &&
              v_cache.is_contiguous() && k_cache.dim() == 4 && v_cache.dim() == 4 &&
              k_cache.size(3) == dim && v_cache.size(0) == k_cache.size(0) &&
              v_cache.size(1) == k_cache.size(1), "cache shape");
  const int kv_heads = k_cache.size(2), v_heads = v_cache.size(2);
  const int vdim = v_cache.size(3), block_size = k_cache.size(1);
  TORCH_CHECK(kv_heads >= 1 && heads % kv_heads == 0 && v_heads >= 1 &&
              kv_heads % v_heads == 0, "head counts");
  TORCH_CHECK(vdim <= 1024, "value size above 1024 is not supported");
  TORCH_CHECK(q.stride(2) == 1 && q.stride(1) == dim && out.stride(2) == 1 &&
              out.stride(1) == vdim && out.size(0) == rows && out.size(1) == heads &&
              out.size(2) == vdim);
  const auto dt = q.scalar_type();
  TORCH_CHECK(k_cache.scalar_type() == dt && v_cache.scalar_type() == dt);
  check_i32(seq_lens, "seq_lens");
  const int nseq = seq_lens.numel();
  TORCH_CHECK(block_tables.is_cuda() &&
              block_tables.scalar_type() == at::ScalarType::Int &&
              block_tables.dim() == 2 && block_tables.stride(1) == 1 &&
              block_tables.size(0) >= nseq);
  const int* qsl = nullptr;
  if (query_start_loc.has_value()) {
    check_i32(query_start_loc.value(), "query_start_loc");
    TORCH_CHECK(query_start_loc.value().numel() == nseq + 1);
    qsl = ptr<int>(query_start_loc.value());
  } else {
    TORCH_CHECK(rows == nseq, "one query row per sequence expected");
  }
  if (rows == 0) return;
  const int elems16 = dt == at::ScalarType::Float ? 4 : 8;
  const int vec_ok = dim % elems16 == 0 && aligned16(k_cache);
  DISPATCH_F32_BF16(dt, {
    launch_chunk_attention<scalar_t>(
        ptr<float>(out), (long)out.stride(0), ptr<scalar_t>(q), (long)q.stride(0),
        ptr<scalar_t>(k_cache), ptr<scalar_t>(v_cache), ptr<int>(block_tables),
        (int)block_tables.stride(0), qsl, ptr<int>(seq_lens), nseq, (float)scale,
        rows, heads, kv_heads, v_heads, dim, vdim, block_size, vec_ok, (int)chunk,
        stream());
  });
}

void diff_combine(torch::Tensor out, torch::Tensor a, double lam, double out_scale,
                  double eps, c10::optional<torch::Tensor> gate) {
  check_f32(a, "a");
  TORCH_CHECK(a.dim() == 4 && a.size(1) == 2, "a is [rows, 2, heads, vdim]");
  const int tokens = a.size(0), heads = a.size(2), vdim = a.size(3);
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() && is_f32_or_bf16(out) &&
              out.numel() == (long)tokens * heads * vdim);
  long g_st = 0;
  if (gate.has_value()) {
    const auto& g = gate.value();
    TORCH_CHECK(g.is_cuda() && g.dim() == 2 && g.size(0) == tokens &&
                g.size(1) == heads && g.stride(1) == 1 &&
                g.scalar_type() == out.scalar_type(), "gate is [rows, heads]");
    g_st = g.stride(0);
  }
  if (tokens == 0) return;
  DISPATCH_F32_BF16(out.scalar_type(), {
    launch_diff_combine<scalar_t>(
        ptr<scalar_t>(out), ptr<float>(a), (float)lam, (float)out_scale, (float)eps,
        gate.has_value() ? ptr<scalar_t>(gate.value()) : nullptr, g_st, tokens, heads,
        vdim, stream());
  });
}

void group_rms_norm(torch::Tensor out, torch::Tensor y, torch::Tensor weight,
                    int64_t groups, double eps) {
  check_f32(weight, "weight");
  TORCH_CHECK(y.is_cuda() && y.is_contiguous() && y.dim() == 2 && is_f32_or_bf16(y));
  const long rows = y.size(0);
  const int width = y.size(1);
  TORCH_CHECK(groups >= 1 && width % groups == 0 && weight.numel() == width);
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() && out.numel() == y.numel() &&
              is_f32_or_bf16(out));
  if (rows == 0) return;
  const int gsize = width / groups;
  const bool in32 = y.scalar_type() == at::ScalarType::Float;
  const bool out32 = out.scalar_type() == at::ScalarType::Float;
  if (in32 && out32)
    launch_group_rms_norm<float, float>(ptr<float>(out), ptr<float>(y),
                                        ptr<float>(weight), (float)eps, rows,
                                        (int)groups, gsize, stream());
  else if (in32)
    launch_group_rms_norm<__hip_bfloat16, float>(
        ptr<__hip_bfloat16>(out), ptr<float>(y), ptr<float>(weight), (float)eps, rows,
        (int)groups, gsize, stream());
  else if (!out32)
    launch_group_rms_norm<__hip_bfloat16, __hip_bfloat16>(
        ptr<__hip_bfloat16>(out), ptr<__hip_bfloat16>(y), ptr<float>(weight),
        (float)eps, rows, (int)groups, gsize, stream());
  else
    TORCH_CHECK(false, "group_rms_norm: bf16 rows give bf16 rows");
}

void hgrn2_scan(torch::Tensor o, torch::Tensor q, torch::Tensor f, torch::Tensor v,
                torch::Tensor f_bias, torch::Tensor lower, torch::Tensor state,
                torch::Tensor loc, torch::Tensor seq_lens, torch::Tensor slots) {
  const int nseq = check_seqs(loc, seq_lens, slots);
  check_f32(o, "o");
  check_f32(f_bias, "f_bias");
  check_f32(lower, "lower");
  check_f32(state, "state");
  check_heads_view(q, "q");
  check_heads_view(f, "f");
  check_heads_view(v, "v");
  const int rows = q.size(0), heads = q.size(1), dim = q.size(2), vdim = v.size(2);
  const auto dt = q.scalar_type();
  TORCH_CHECK(f.sizes() == q.sizes() && v.size(0) == rows && v.size(1) == heads &&
              f.scalar_type() == dt && v.scalar_type() == dt);
  TORCH_CHECK(dim >= 1 && dim <= 1024, "hgrn2_scan: head size");
  TORCH_CHECK(f_bias.numel() == (long)heads * dim && lower.numel() == (long)heads * dim);
  TORCH_CHECK(o.numel() == (long)rows * heads * vdim);
  TORCH_CHECK(state.dim() == 4 && state.size(1) == heads && state.size(2) == vdim &&
              state.size(3) == dim, "hgrn2_scan: state must be [slots, heads, vdim, dim]");
  if (rows == 0 || nseq == 0) return;
  // gate and activated query per (row, head, channel), f32
  auto gq = torch::empty({(long)rows, 2L * heads * dim}, o.options());
  const int vec_ok = dim % 4 == 0 && aligned16(state) && aligned16(gq);
  DISPATCH_F32_BF16(dt, {
    launch_hgrn2_scan<scalar_t>(
        ptr<float>(o), ptr<scalar_t>(q), (long)q.stride(0), ptr<scalar_t>(f),
        (long)f.stride(0), ptr<scalar_t>(v), (long)v.stride(0), ptr<float>(f_bias),
        ptr<float>(lower), ptr<float>(state), ptr<int>(loc), ptr<int>(seq_lens),
        ptr<int>(slots), nseq, heads, dim, vdim, vec_ok, ptr<float>(gq), rows,
        stream());
  });
}

void silu_mul_scaled(torch::Tensor out, torch::Tensor gu, torch::Tensor scale) {
  check_f32(scale, "col_scale");
  TORCH_CHECK(gu.is_cuda() && gu.is_contiguous() && gu.dim() == 2 &&
              is_f32_or_bf16(gu) && scale.dim() == 2 && scale.size(0) == gu.size(0));
  const long tokens = gu.size(0);
  const int experts = scale.size(1);
  TORCH_CHECK(experts >= 1 && gu.size(1) % (2 * experts) == 0);
  const int ff = gu.size(1) / (2 * experts);
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() &&
              out.scalar_type() == gu.scalar_type() &&
              out.numel() == tokens * experts * ff);
  if (tokens == 0) return;
  DISPATCH_F32_BF16(gu.scalar_type(), {
    launch_silu_mul_scaled<scalar_t>(ptr<scalar_t>(out), ptr<scalar_t>(gu),
                                     ptr<float>(scale), tokens, experts, ff, stream());
  });
}

}  // namespace

void register_mix_ops(pybind11::module& m) {
  m.def("token_shift_state", &token_shift_state);
  m.def("qk_norm_rope_cache_write", &qk_norm_rope_cache_write);
  m.def("chunk_attention", &chunk_attention);
  m.def("diff_combine", &diff_combine);
  m.def("group_rms_norm", &group_rms_norm);
  m.def("hgrn2_scan", &hgrn2_scan);
  m.def("silu_mul_scaled", &silu_mul_scaled);
}
