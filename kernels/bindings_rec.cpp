// Torch bindings (part of `_C_seq`): layer norms of the f32 stream, query/key
// norm with cache write, grouped-query attention of any shape, gated group
// norm, and the recurrences with per-sequence state.  Every shape the kernels
// assume is checked here, on the host, before a launch.

#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>

#include <hip/hip_bf16.h>

template <typename T>
void launch_layer_norm_stream(T*, const float*, const float*, float, int, int,
                              hipStream_t);
template <typename T>
void launch_stream_add_layer_norm(float*, const T*, const T*, float, float,
                                  const float*, const float*, float, int, int,
                                  T*, const float*, float, hipStream_t);
void launch_stream_add_vec(float*, const float*, const float*, int, long,
                           hipStream_t);
template <typename T>
void launch_gated_group_norm(T*, const float*, const T*, long, const float*,
                             float, int, int, int, int, hipStream_t);
template <typename T>
void launch_qk_norm_cache_write(T*, const T*, long, const T*, long, const T*,
                                long, const float*, const float*, float,
                                const long*, float, int, T*, T*, const long*,
                                int, int, int, int, int, hipStream_t);
template <typename T>
void launch_paged_attention_any(T*, long, const T*, long, const T*, const T*,
                                const int*, int, const int*, const int*, int,
                                float, int, int, int, int, int, int, int, int,
                                int, float, hipStream_t);
template <typename T>
void launch_ssd_scan(float*, const T*, long, const T*, long, const float*,
                     const float*, const float*, float*, const int*, const int*,
                     const int*, int, int, int, int, int, int, float*, int,
                     hipStream_t);
template <typename T>
void launch_mlstm_scan(float*, const T*, long, const T*, long, const T*, long,
                       const T*, long, const T*, long, const float*,
                       const float*, float, float, float*, float*, float*,
                       const int*, const int*, const int*, int, int, int, int,
                       int, float*, int, hipStream_t);
template <typename T>
void launch_rglru_scan(T*, const T*, const T*, const T*, const float*,
                       const float*, const float*, float, const T*, float*,
                       const int*, const int*, const int*, int, int,
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

// rows of each sequence, its length and its slot; returns the sequence count
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

void layer_norm_stream(torch::Tensor out, torch::Tensor x, torch::Tensor weight,
                       double eps) {
  check_f32(x, "x");
  check_f32(weight, "weight");
  const int width = x.size(-1);
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() && out.numel() == x.numel() &&
              weight.numel() == width);
  const int rows = x.numel() / width;
  DISPATCH_F32_BF16(out.scalar_type(), {
    launch_layer_norm_stream<scalar_t>(ptr<scalar_t>(out), ptr<float>(x),
                                       ptr<float>(weight), (float)eps, rows,
                                       width, stream());
  });
}

void stream_add_layer_norm(torch::Tensor x, torch::Tensor a,
                           c10::optional<torch::Tensor> b, double sa, double sb,
                           torch::Tensor weight,
                           c10::optional<torch::Tensor> layer_scale, double eps,
                           c10::optional<torch::Tensor> next_out,
                           c10::optional<torch::Tensor> next_weight,
                           double next_eps) {
  check_f32(x, "x");
  check_f32(weight, "weight");
  const int width = x.size(-1);
  TORCH_CHECK(a.is_cuda() && a.is_contiguous() && a.numel() == x.numel() &&
              weight.numel() == width);
  if (b.has_value())
    TORCH_CHECK(b.value().is_cuda() && b.value().is_contiguous() &&
                b.value().numel() == x.numel() &&
                b.value().scalar_type() == a.scalar_type());
  if (layer_scale.has_value()) {
    check_f32(layer_scale.value(), "layer_scale");
    TORCH_CHECK(layer_scale.value().numel() == width);
  }
  TORCH_CHECK(next_out.has_value() == next_weight.has_value());
  if (next_out.has_value()) {
    check_f32(next_weight.value(), "next_weight");
    TORCH_CHECK(next_weight.value().numel() == width &&
                next_out.value().is_cuda() && next_out.value().is_contiguous() &&
                next_out.value().numel() == x.numel() &&
                next_out.value().scalar_type() == a.scalar_type());
  }
  const int rows = x.numel() / width;
  DISPATCH_F32_BF16(a.scalar_type(), {
    launch_stream_add_layer_norm<scalar_t>(
        ptr<float>(x), ptr<scalar_t>(a),
        b.has_value() ? ptr<scalar_t>(b.value()) : nullptr, (float)sa, (float)sb,
        ptr<float>(weight),
        layer_scale.has_value() ? ptr<float>(layer_scale.value()) : nullptr,
        (float)eps, rows, width,
        next_out.has_value() ? ptr<scalar_t>(next_out.value()) : nullptr,
        next_out.has_value() ? ptr<float>(next_weight.value()) : nullptr,
        (float)next_eps, stream());
  });
}

void stream_add_vec(torch::Tensor x, c10::optional<torch::Tensor> other,
                    torch::Tensor vec) {
  check_f32(x, "x");
  check_f32(vec, "vec");
  const int width = x.size(-1);
  TORCH_CHECK(vec.numel() == width);
  if (other.has_value()) {
    check_f32(other.value(), "other");
    TORCH_CHECK(other.value().numel() == x.numel());
  }
  launch_stream_add_vec(ptr<float>(x),
                        other.has_value() ? ptr<float>(other.value()) : nullptr,
                        ptr<float>(vec), width, x.numel(), stream());
}

void gated_group_norm(torch::Tensor out, torch::Tensor y, torch::Tensor gate,
                      torch::Tensor weight, int64_t groups, double eps,
                      bool gate_first) {
  check_f32(y, "y");
  check_f32(weight, "weight");
  TORCH_CHECK(y.dim() == 2 && gate.dim() == 2 && gate.is_cuda() &&
              gate.stride(1) == 1 && gate.size(0) == y.size(0) &&
              gate.size(1) == y.size(1));
  const int rows = y.size(0), cols = y.size(1);
  TORCH_CHECK(groups >= 1 && cols % groups == 0 && weight.numel() == cols);
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() && out.numel() == y.numel() &&
              out.scalar_type() == gate.scalar_type());
  DISPATCH_F32_BF16(gate.scalar_type(), {
    launch_gated_group_norm<scalar_t>(
        ptr<scalar_t>(out), ptr<float>(y), ptr<scalar_t>(gate),
        (long)gate.stride(0), ptr<float>(weight), (float)eps, rows, cols,
        (int)groups, gate_first ? 1 : 0, stream());
  });
}

void qk_norm_cache_write(torch::Tensor q_out, torch::Tensor q, torch::Tensor k,
                         torch::Tensor v, torch::Tensor q_weight,
                         torch::Tensor k_weight, double eps,
                         torch::Tensor positions, double temp_coef,
                         int64_t temp_every, torch::Tensor k_cache,
                         torch::Tensor v_cache, torch::Tensor slot_mapping) {
  TORCH_CHECK(q.is_cuda() && q.dim() == 3 && k.dim() == 3 && v.dim() == 3);
  const int tokens = q.size(0), heads = q.size(1), dim = q.size(2);
  const int kv_heads = k.size(1), vdim = v.size(2);
  TORCH_CHECK(k.size(0) == tokens && v.size(0) == tokens && k.size(2) == dim &&
              v.size(1) == kv_heads);
  // heads lie side by side within a row; rows may be strided
  TORCH_CHECK(q.stride(2) == 1 && q.stride(1) == dim && k.stride(2) == 1 &&
              k.stride(1) == dim && v.stride(2) == 1 && v.stride(1) == vdim);
  check_f32(q_weight, "q_weight");
  check_f32(k_weight, "k_weight");
  TORCH_CHECK(q_weight.numel() == dim && k_weight.numel() == dim);
  check_i64(positions, "positions");
  check_i64(slot_mapping, "slot_mapping");
  TORCH_CHECK(positions.numel() == tokens && slot_mapping.numel() == tokens);
  TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous() &&
              k_cache.dim() == 4 && v_cache.dim() == 4 &&
              k_cache.size(2) == kv_heads && k_cache.size(3) == dim &&
              v_cache.size(2) == kv_heads && v_cache.size(3) == vdim &&
              v_cache.size(0) == k_cache.size(0) &&
              v_cache.size(1) == k_cache.size(1), "cache shape");
  TORCH_CHECK(q_out.is_contiguous() && q_out.numel() == q.numel());
  const auto dt = q.scalar_type();
  TORCH_CHECK(k.scalar_type() == dt && v.scalar_type() == dt &&
              q_out.scalar_type() == dt && k_cache.scalar_type() == dt &&
              v_cache.scalar_type() == dt);
  DISPATCH_F32_BF16(dt, {
    launch_qk_norm_cache_write<scalar_t>(
        ptr<scalar_t>(q_out), ptr<scalar_t>(q), (long)q.stride(0),
        ptr<scalar_t>(k), (long)k.stride(0), ptr<scalar_t>(v), (long)v.stride(0),
        ptr<float>(q_weight), ptr<float>(k_weight), (float)eps,
        ptr<long>(positions), (float)temp_coef, (int)temp_every,
        ptr<scalar_t>(k_cache), ptr<scalar_t>(v_cache), ptr<long>(slot_mapping),
        tokens, heads, kv_heads, dim, vdim, stream());
  });
}

void paged_attention_any(torch::Tensor out, torch::Tensor q, torch::Tensor k_cache,
                         torch::Tensor v_cache, torch::Tensor block_tables,
                         c10::optional<torch::Tensor> query_start_loc,
                         torch::Tensor seq_lens, double scale,
                         int64_t max_query_len, int64_t window, bool has_sink,
                         double sink) {
  TORCH_CHECK(q.is_cuda() && q.dim() == 3 && out.dim() == 3);
  TORCH_CHECK(window >= 0, "window");
  const int rows = q.size(0), heads = q.size(1), dim = q.size(2);
  TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous() &&
              k_cache.dim() == 4 && v_cache.dim() == 4 && k_cache.size(3) == dim &&
              v_cache.size(0) == k_cache.size(0) &&
              v_cache.size(1) == k_cache.size(1) &&
              v_cache.size(2) == k_cache.size(2), "cache shape");
  const int kv_heads = k_cache.size(2), vdim = v_cache.size(3);
  const int block_size = k_cache.size(1);
  TORCH_CHECK(kv_heads >= 1 && heads % kv_heads == 0);
  TORCH_CHECK(vdim <= 1024, "value size above 1024 is not supported");
  TORCH_CHECK(q.stride(2) == 1 && q.stride(1) == dim && out.stride(2) == 1 &&
              out.stride(1) == vdim && out.size(0) == rows &&
              out.size(1) == heads && out.size(2) == vdim);
  const auto dt = q.scalar_type();
  TORCH_CHECK(out.scalar_type() == dt && k_cache.scalar_type() == dt &&
              v_cache.scalar_type() == dt);
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
    launch_paged_attention_any<scalar_t>(
        ptr<scalar_t>(out), (long)out.stride(0), ptr<scalar_t>(q),
        (long)q.stride(0), ptr<scalar_t>(k_cache), ptr<scalar_t>(v_cache),
        ptr<int>(block_tables), (int)block_tables.stride(0), qsl,
        ptr<int>(seq_lens), nseq, (float)scale, rows, heads, kv_heads, dim, vdim,
        block_size, vec_ok, (int)window, has_sink ? 1 : 0, (float)sink, stream());
  });
}

void ssd_scan(torch::Tensor y, torch::Tensor xbc, torch::Tensor dt,
              torch::Tensor dt_bias, torch::Tensor a_log, torch::Tensor d_skip,
              torch::Tensor state, torch::Tensor loc, torch::Tensor seq_lens,
              torch::Tensor slots, int64_t heads, int64_t vdim, int64_t nstate,
              int64_t groups) {
  const int nseq = check_seqs(loc, seq_lens, slots);
  check_f32(y, "y");
  check_f32(dt_bias, "dt_bias");
  check_f32(a_log, "a_log");
  check_f32(d_skip, "d_skip");
  check_f32(state, "state");
  const long inner = heads * vdim;
  TORCH_CHECK(heads >= 1 && groups >= 1 && heads % groups == 0 && nstate >= 1 &&
              nstate <= 1024, "ssd_scan: heads/groups/state sizes");
  TORCH_CHECK(xbc.is_cuda() && xbc.dim() == 2 && xbc.stride(1) == 1 &&
              xbc.size(1) == inner + 2 * groups * nstate, "ssd_scan: xbc width");
  const int rows = xbc.size(0);
  TORCH_CHECK(dt.dim() == 2 && dt.size(0) == rows && dt.size(1) == heads &&
              dt.stride(1) == 1 && dt.scalar_type() == xbc.scalar_type());
  TORCH_CHECK(y.numel() == rows * inner);
  TORCH_CHECK(dt_bias.numel() == heads && a_log.numel() == heads &&
              d_skip.numel() == heads);
  TORCH_CHECK(state.dim() == 4 && state.size(1) == heads &&
              state.size(2) == vdim && state.size(3) == nstate,
              "ssd_scan: state must be [slots, heads, vdim, state]");
  if (rows == 0 || nseq == 0) return;
  const int vec_ok = nstate % 8 == 0 && inner % 8 == 0 && xbc.stride(0) % 8 == 0 &&
                     aligned16(xbc) && aligned16(state);
  // alpha, beta per (row, head), written by the gate kernel ahead of the scan
  auto gates = torch::empty({(long)rows * heads * 4}, y.options());
  DISPATCH_F32_BF16(xbc.scalar_type(), {
    launch_ssd_scan<scalar_t>(
        ptr<float>(y), ptr<scalar_t>(xbc), (long)xbc.stride(0), ptr<scalar_t>(dt),
        (long)dt.stride(0), ptr<float>(dt_bias), ptr<float>(a_log),
        ptr<float>(d_skip), ptr<float>(state), ptr<int>(loc), ptr<int>(seq_lens),
        ptr<int>(slots), nseq, (int)heads, (int)vdim, (int)nstate, (int)groups,
        vec_ok, ptr<float>(gates), rows, stream());
  });
}

void mlstm_scan(torch::Tensor o, torch::Tensor q, torch::Tensor k, torch::Tensor v,
                torch::Tensor i_pre, torch::Tensor f_pre, torch::Tensor i_bias,
                torch::Tensor f_bias, double cap, double q_scale,
                torch::Tensor s_state, torch::Tensor n_state,
                torch::Tensor m_state, torch::Tensor loc, torch::Tensor seq_lens,
                torch::Tensor slots) {
  const int nseq = check_seqs(loc, seq_lens, slots);
  check_f32(o, "o");
  check_f32(i_bias, "i_bias");
  check_f32(f_bias, "f_bias");
  check_f32(s_state, "s_state");
  check_f32(n_state, "n_state");
  check_f32(m_state, "m_state");
  TORCH_CHECK(q.is_cuda() && q.dim() == 3 && k.dim() == 3 && v.dim() == 3);
  const int rows = q.size(0), heads = q.size(1), dim = q.size(2), vdim = v.size(2);
  TORCH_CHECK(dim >= 1 && dim <= 1024, "mlstm_scan: key size above 1024");
  TORCH_CHECK(k.size(0) == rows && k.size(1) == heads && k.size(2) == dim &&
              v.size(0) == rows && v.size(1) == heads);
  TORCH_CHECK(q.stride(2) == 1 && q.stride(1) == dim && k.stride(2) == 1 &&
              k.stride(1) == dim && v.stride(2) == 1 && v.stride(1) == vdim);
  TORCH_CHECK(i_pre.dim() == 2 && f_pre.dim() == 2 && i_pre.size(0) == rows &&
              f_pre.size(0) == rows && i_pre.size(1) == heads &&
              f_pre.size(1) == heads && i_pre.stride(1) == 1 &&
              f_pre.stride(1) == 1);
  const auto dt = q.scalar_type();
  TORCH_CHECK(k.scalar_type() == dt && v.scalar_type() == dt &&
              i_pre.scalar_type() == dt && f_pre.scalar_type() == dt);
  TORCH_CHECK(i_bias.numel() == heads && f_bias.numel() == heads);
  TORCH_CHECK(o.numel() == (long)rows * heads * vdim);
  TORCH_CHECK(s_state.dim() == 4 && s_state.size(1) == heads &&
              s_state.size(2) == vdim && s_state.size(3) == dim,
              "mlstm_scan: S must be [slots, heads, vdim, dim]");
  TORCH_CHECK(n_state.dim() == 3 && n_state.size(0) == s_state.size(0) &&
              n_state.size(1) == heads && n_state.size(2) == dim &&
              m_state.dim() == 2 && m_state.size(0) == s_state.size(0) &&
              m_state.size(1) == heads);
  if (rows == 0 || nseq == 0) return;
  const int vec_ok = dim % 8 == 0 && q.stride(0) % 8 == 0 && k.stride(0) % 8 == 0 &&
                     aligned16(q) && aligned16(k) && aligned16(s_state) &&
                     aligned16(n_state);
  // alpha, beta, exp(-m) per (row, head), written by the gate kernels
  auto gates = torch::empty({(long)rows * heads * 4}, o.options());
  DISPATCH_F32_BF16(dt, {
    launch_mlstm_scan<scalar_t>(
        ptr<float>(o), ptr<scalar_t>(q), (long)q.stride(0), ptr<scalar_t>(k),
        (long)k.stride(0), ptr<scalar_t>(v), (long)v.stride(0),
        ptr<scalar_t>(i_pre), (long)i_pre.stride(0), ptr<scalar_t>(f_pre),
        (long)f_pre.stride(0), ptr<float>(i_bias), ptr<float>(f_bias), (float)cap,
        (float)q_scale, ptr<float>(s_state), ptr<float>(n_state),
        ptr<float>(m_state), ptr<int>(loc), ptr<int>(seq_lens), ptr<int>(slots),
        nseq, heads, dim, vdim, vec_ok, ptr<float>(gates), rows, stream());
  });
}

void rglru_scan(torch::Tensor out, torch::Tensor u, torch::Tensor r_pre,
                torch::Tensor i_pre, torch::Tensor r_bias, torch::Tensor i_bias,
                torch::Tensor lam, double gate_c, torch::Tensor y_branch,
                torch::Tensor state, torch::Tensor loc, torch::Tensor seq_lens,
                torch::Tensor slots) {
  const int nseq = check_seqs(loc, seq_lens, slots);
  check_f32(r_bias, "r_bias");
  check_f32(i_bias, "i_bias");
  check_f32(lam, "lam");
  check_f32(state, "state");
  TORCH_CHECK(u.is_cuda() && u.dim() == 2 && u.is_contiguous());
  const int rows = u.size(0), width = u.size(1);
  const auto dt = u.scalar_type();
  for (const torch::Tensor* t : {&out, &r_pre, &i_pre, &y_branch})
    TORCH_CHECK(t->is_cuda() && t->is_contiguous() && t->scalar_type() == dt &&
                t->numel() == u.numel(), "rglru_scan: row tensors must match u");
  TORCH_CHECK(r_bias.numel() == width && i_bias.numel() == width &&
              lam.numel() == width);
  TORCH_CHECK(state.dim() == 2 && state.size(1) == width);
  if (rows == 0 || nseq == 0) return;
  DISPATCH_F32_BF16(dt, {
    launch_rglru_scan<scalar_t>(
        ptr<scalar_t>(out), ptr<scalar_t>(u), ptr<scalar_t>(r_pre),
        ptr<scalar_t>(i_pre), ptr<float>(r_bias), ptr<float>(i_bias),
        ptr<float>(lam), (float)gate_c, ptr<scalar_t>(y_branch),
        ptr<float>(state), ptr<int>(loc), ptr<int>(seq_lens), ptr<int>(slots),
        nseq, width, stream());
  });
}

}  // namespace

void register_rec_ops(pybind11::module& m) {
  m.def("layer_norm_stream", &layer_norm_stream);
  m.def("stream_add_layer_norm", &stream_add_layer_norm);
  m.def("stream_add_vec", &stream_add_vec);
  m.def("gated_group_norm", &gated_group_norm);
  m.def("qk_norm_cache_write", &qk_norm_cache_write);
  m.def("paged_attention_any", &paged_attention_any);
  m.def("ssd_scan", &ssd_scan);
  m.def("mlstm_scan", &mlstm_scan);
  m.def("rglru_scan", &rglru_scan);
}
