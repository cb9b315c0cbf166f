// Torch bindings of the two-norm residual kernel, rotation + cache write,
// output gates, squared relu, expert router / combine and the grouped expert
// product (part of the `_C_seq` extension; registered from bindings_seq.cpp).

#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>

#include <hip/hip_bf16.h>

template <typename T>
void launch_stream_add_rms_norm_pair(float*, const T*, const T*, const float*,
                                     const T*, const float*, const float*, float,
                                     int, int, T*, T*, hipStream_t);
template <typename T>
void launch_rope_kv_cache_write(T*, const T*, long, const T*, long, const T*,
                                long, const long*, const float*, int, int, float,
                                T*, T*, const long*, int, int, int, int, int,
                                hipStream_t);
template <typename T>
void launch_sigmoid_gate_mul(T*, const T*, long, long, const T*, long, long, int,
                             int, int, int, hipStream_t);
template <typename T>
void launch_relu2(T*, const T*, long, const T*, const float*, int, int, int,
                  hipStream_t);
int moe_route_max_experts();
void launch_moe_route(float*, float*, int*, float*, const float*, const float*,
                      int, int, int, int, int, hipStream_t);
template <typename T>
void launch_moe_combine(T*, const T*, const int*, const int*, const float*, int,
                        int, int, int, hipStream_t);
int moe_sort_max_experts();
template <typename T>
void launch_moe_sort(T*, int*, int*, int*, const T*, long, const int*, int, int,
                     int, int, const float*, hipStream_t);
void launch_moe_gemm(__hip_bfloat16*, const __hip_bfloat16*,
                     const __hip_bfloat16*, const int*, int, int, int, int, int,
                     hipStream_t);

namespace {

hipStream_t stream() { return at::hip::getCurrentHIPStream().stream(); }

template <typename T>
T* ptr(const torch::Tensor& t) {
  return reinterpret_cast<T*>(t.data_ptr());
}
template <typename T>
T* optr(const c10::optional<torch::Tensor>& t) {
  return t.has_value() ? reinterpret_cast<T*>(t.value().data_ptr()) : nullptr;
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

// an optional [rows, width] tensor of the compute type
void check_rows(const c10::optional<torch::Tensor>& t, at::ScalarType dt, long rows,
                long width, const char* what) {
  if (!t.has_value()) return;
  const auto& v = t.value();
  TORCH_CHECK(v.is_cuda() && v.is_contiguous() && v.scalar_type() == dt &&
                  v.dim() == 2 && v.size(0) == rows && v.size(1) == width,
              what, ": expected a contiguous [rows, width] tensor of the compute type");
}

void stream_add_rms_norm_pair(torch::Tensor x, c10::optional<torch::Tensor> a,
                              c10::optional<torch::Tensor> b,
                              c10::optional<torch::Tensor> row_scale,
                              c10::optional<torch::Tensor> c,
                              c10::optional<torch::Tensor> w1,
                              c10::optional<torch::Tensor> w2, double eps,
                              c10::optional<torch::Tensor> h1,
                              c10::optional<torch::Tensor> h2) {
  check_f32(x, "x");
  TORCH_CHECK(x.dim() == 2);
  const long rows = x.size(0), width = x.size(1);
  TORCH_CHECK(a.has_value() || (!b.has_value() && !c.has_value()),
              "b and c need a");
  TORCH_CHECK(c.has_value() == row_scale.has_value(), "c and row_scale go together");
  TORCH_CHECK(w1.has_value() == h1.has_value() && w2.has_value() == h2.has_value(),
              "a norm weight needs its output");
  at::ScalarType dt;
  if (a.has_value()) dt = a.value().scalar_type();
  else if (h1.has_value()) dt = h1.value().scalar_type();
  else if (h2.has_value()) dt = h2.value().scalar_type();
  else return;
  check_rows(a, dt, rows, width, "a");
  check_rows(b, dt, rows, width, "b");
  check_rows(c, dt, rows, width, "c");
  check_rows(h1, dt, rows, width, "h1");
  check_rows(h2, dt, rows, width, "h2");
  if (row_scale.has_value()) {
    check_f32(row_scale.value(), "row_scale");
    TORCH_CHECK(row_scale.value().numel() == rows);
  }
  for (const auto* w : {&w1, &w2})
    if (w->has_value()) {
      check_f32(w->value(), "norm weight");
      TORCH_CHECK(w->value().numel() == width);
    }
  if (rows == 0) return;
  DISPATCH_F32_BF16(dt, {
    launch_stream_add_rms_norm_pair<scalar_t>(
        ptr<float>(x), optr<scalar_t>(a), optr<scalar_t>(b), optr<float>(row_scale),
        optr<scalar_t>(c), optr<float>(w1), optr<float>(w2), (float)eps, (int)rows,
        (int)width, optr<scalar_t>(h1), optr<scalar_t>(h2), stream());
  });
}

void rope_kv_cache_write(torch::Tensor q_out, torch::Tensor q, torch::Tensor k,
                         torch::Tensor v, torch::Tensor positions,
                         torch::Tensor inv_freq, int64_t rot_dims, bool interleaved,
                         double mag, torch::Tensor k_cache, torch::Tensor v_cache,
                         torch::Tensor slot_mapping) {
  TORCH_CHECK(q.is_cuda() && q.dim() == 3 && k.dim() == 3 && v.dim() == 3);
  const int tokens = q.size(0), heads = q.size(1), dim = q.size(2);
  const int kv_heads = k.size(1), vdim = v.size(2);
  TORCH_CHECK(k.size(0) == tokens && v.size(0) == tokens && k.size(2) == dim &&
              v.size(1) == kv_heads, "q / k / v shapes");
  TORCH_CHECK(q.stride(2) == 1 && q.stride(1) == dim && k.stride(2) == 1 &&
              k.stride(1) == dim && v.stride(2) == 1 && v.stride(1) == vdim,
              "heads must be dense within a row");
  TORCH_CHECK(q_out.is_contiguous() && q_out.sizes() == q.sizes());
  const auto dt = q.scalar_type();
  TORCH_CHECK(k.scalar_type() == dt && v.scalar_type() == dt &&
              q_out.scalar_type() == dt && k_cache.scalar_type() == dt &&
              v_cache.scalar_type() == dt);
  TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous() &&
              k_cache.dim() == 4 && v_cache.dim() == 4 &&
              k_cache.size(2) == kv_heads && k_cache.size(3) == dim &&
              v_cache.size(0) == k_cache.size(0) && v_cache.size(1) == k_cache.size(1) &&
              v_cache.size(2) == kv_heads && v_cache.size(3) == vdim, "cache shape");
  check_i64(positions, "positions");
  check_i64(slot_mapping, "slot_mapping");
  check_f32(inv_freq, "inv_freq");
  TORCH_CHECK(positions.numel() == tokens && slot_mapping.numel() == tokens);
  TORCH_CHECK(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= dim &&
              inv_freq.numel() >= rot_dims / 2, "rot_dims");
  if (tokens == 0) return;
  DISPATCH_F32_BF16(dt, {
    launch_rope_kv_cache_write<scalar_t>(
        ptr<scalar_t>(q_out), ptr<scalar_t>(q), (long)q.stride(0), ptr<scalar_t>(k),
        (long)k.stride(0), ptr<scalar_t>(v), (long)v.stride(0), ptr<long>(positions),
        ptr<float>(inv_freq), (int)(rot_dims / 2), interleaved ? 1 : 0, (float)mag,
        ptr<scalar_t>(k_cache), ptr<scalar_t>(v_cache), ptr<long>(slot_mapping),
        tokens, heads, kv_heads, dim, vdim, stream());
  });
}

void sigmoid_gate_mul(torch::Tensor out, torch::Tensor o, torch::Tensor gate) {
  TORCH_CHECK(o.is_cuda() && o.dim() == 3 && o.stride(2) == 1);
  const int tokens = o.size(0), heads = o.size(1), d = o.size(2);
  TORCH_CHECK(out.is_contiguous() && out.numel() == o.numel() &&
              out.scalar_type() == o.scalar_type() &&
              gate.scalar_type() == o.scalar_type());
  const bool per_head = gate.dim() == 2;
  if (per_head) {
    TORCH_CHECK(gate.size(0) == tokens && gate.size(1) == heads && gate.stride(1) == 1);
  } else {
    TORCH_CHECK(gate.dim() == 3 && gate.size(0) == tokens && gate.size(1) == heads &&
                gate.size(2) == d && gate.stride(2) == 1);
  }
  if (o.numel() == 0) return;
  DISPATCH_F32_BF16(o.scalar_type(), {
    launch_sigmoid_gate_mul<scalar_t>(
        ptr<scalar_t>(out), ptr<scalar_t>(o), (long)o.stride(0), (long)o.stride(1),
        ptr<scalar_t>(gate), (long)gate.stride(0), per_head ? 1L : (long)gate.stride(1),
        per_head ? 1 : 0, tokens, heads, d, stream());
  });
}

void relu2(torch::Tensor out, torch::Tensor x, c10::optional<torch::Tensor> bias,
           c10::optional<torch::Tensor> col_scale) {
  TORCH_CHECK(x.is_cuda() && x.dim() == 2 && x.stride(1) == 1);
  const int rows = x.size(0), cols = x.size(1);
  TORCH_CHECK(out.is_contiguous() && out.numel() == x.numel() &&
              out.scalar_type() == x.scalar_type());
  if (bias.has_value())
    TORCH_CHECK(bias.value().is_contiguous() && bias.value().numel() == cols &&
                bias.value().scalar_type() == x.scalar_type(), "bias");
  int nscale = 0;
  if (col_scale.has_value()) {
    check_f32(col_scale.value(), "col_scale");
    TORCH_CHECK(col_scale.value().dim() == 2 && col_scale.value().size(0) == rows);
    nscale = col_scale.value().size(1);
    TORCH_CHECK(nscale >= 1 && cols % nscale == 0, "columns must divide into the scale's blocks");
  }
  if (x.numel() == 0) return;
  DISPATCH_F32_BF16(x.scalar_type(), {
    launch_relu2<scalar_t>(ptr<scalar_t>(out), ptr<scalar_t>(x), (long)x.stride(0),
                           optr<scalar_t>(bias), optr<float>(col_scale), nscale, rows,
                           cols, stream());
  });
}

void moe_route(torch::Tensor dense, torch::Tensor ident, torch::Tensor ids,
               torch::Tensor wts, torch::Tensor logits, torch::Tensor correction,
               int64_t num_real) {
  check_f32(logits, "logits");
  check_f32(correction, "correction");
  check_f32(dense, "dense");
  check_f32(ident, "identity");
  check_f32(wts, "weights");
  check_i32(ids, "ids");
  TORCH_CHECK(logits.dim() == 2 && ids.dim() == 2);
  const int tokens = logits.size(0), n = logits.size(1), top = ids.size(1);
  TORCH_CHECK(n <= moe_route_max_experts(), "too many router outputs");
  TORCH_CHECK(correction.numel() == n && num_real >= 0 && num_real <= n &&
              top >= 1 && top <= n);
  TORCH_CHECK(ids.size(0) == tokens && wts.dim() == 2 && wts.size(0) == tokens &&
              wts.size(1) == top && ident.numel() == tokens &&
              dense.numel() == (long)tokens * num_real);
  if (tokens == 0) return;
  launch_moe_route(ptr<float>(dense), ptr<float>(ident), ptr<int>(ids), ptr<float>(wts),
                   ptr<float>(logits), ptr<float>(correction), tokens, n, (int)num_real,
                   top, 0, stream());
}

// sigmoid scores, the top ones as they are (no correction, no renormalising)
void moe_route_sigmoid(torch::Tensor dense, torch::Tensor ids, torch::Tensor wts,
                       torch::Tensor logits) {
  check_f32(logits, "logits");
  check_f32(dense, "dense");
  check_f32(wts, "weights");
  check_i32(ids, "ids");
  TORCH_CHECK(logits.dim() == 2 && ids.dim() == 2);
  const int tokens = logits.size(0), n = logits.size(1), top = ids.size(1);
  TORCH_CHECK(n <= moe_route_max_experts(), "too many router outputs");
  TORCH_CHECK(top >= 1 && top <= n && ids.size(0) == tokens && wts.dim() == 2 &&
              wts.size(0) == tokens && wts.size(1) == top &&
              dense.numel() == (long)tokens * n);
  if (tokens == 0) return;
  launch_moe_route(ptr<float>(dense), nullptr, ptr<int>(ids), ptr<float>(wts),
                   ptr<float>(logits), nullptr, tokens, n, n, top, 1, stream());
}

void moe_combine(torch::Tensor out, torch::Tensor ye, torch::Tensor pos,
                 torch::Tensor ids, torch::Tensor wts, int64_t num_real) {
  check_i32(pos, "pos");
  check_i32(ids, "ids");
  check_f32(wts, "weights");
  TORCH_CHECK(ye.is_cuda() && ye.is_contiguous() && ye.dim() == 2 &&
              out.is_contiguous() && out.dim() == 2 && out.size(1) == ye.size(1) &&
              out.scalar_type() == ye.scalar_type());
  const int tokens = out.size(0), top = ids.size(1), width = out.size(1);
  TORCH_CHECK(ids.size(0) == tokens && pos.sizes() == ids.sizes() &&
              wts.sizes() == ids.sizes() && ye.size(0) >= (long)tokens * top);
  if (out.numel() == 0) return;
  DISPATCH_F32_BF16(ye.scalar_type(), {
    launch_moe_combine<scalar_t>(ptr<scalar_t>(out), ptr<scalar_t>(ye), ptr<int>(pos),
                                 ptr<int>(ids), ptr<float>(wts), tokens, top,
                                 (int)num_real, width, stream());
  });
}

void moe_sort(torch::Tensor xs, torch::Tensor pos, torch::Tensor seg,
              torch::Tensor scratch, torch::Tensor h, torch::Tensor ids,
              int64_t num_real, c10::optional<torch::Tensor> row_scale) {
  check_i32(ids, "ids");
  check_i32(pos, "pos");
  check_i32(seg, "seg");
  check_i32(scratch, "scratch");
  TORCH_CHECK(h.is_cuda() && h.dim() == 2 && h.stride(1) == 1 && ids.dim() == 2 &&
              ids.size(0) == h.size(0));
  const int tokens = h.size(0), width = h.size(1), top = ids.size(1);
  TORCH_CHECK(num_real >= 1 && num_real <= moe_sort_max_experts(), "number of experts");
  TORCH_CHECK(pos.sizes() == ids.sizes() && seg.numel() == num_real + 1 &&
              scratch.numel() == 2 * num_real);
  TORCH_CHECK(xs.is_contiguous() && xs.dim() == 2 && xs.size(0) == (long)tokens * top &&
              xs.size(1) == width && xs.scalar_type() == h.scalar_type());
  if (row_scale.has_value()) {
    check_f32(row_scale.value(), "row_scale");
    TORCH_CHECK(row_scale.value().sizes() == ids.sizes(), "row_scale is [tokens, top]");
  }
  if (tokens == 0) return;
  DISPATCH_F32_BF16(h.scalar_type(), {
    launch_moe_sort<scalar_t>(ptr<scalar_t>(xs), ptr<int>(pos), ptr<int>(seg),
                              ptr<int>(scratch), ptr<scalar_t>(h), (long)h.stride(0),
                              ptr<int>(ids), tokens, top, (int)num_real, width,
                              optr<float>(row_scale), stream());
  });
}

// mode 0: plain, 1: silu(first half) * second half, 2: squared relu
void moe_gemm(torch::Tensor y, torch::Tensor x, torch::Tensor w,
              torch::Tensor seg_off, int64_t mode) {
  const int T = x.size(0);
  const int K = x.size(1);
  const int E = w.size(0);
  const long wn = w.size(1);
  const int N = mode == 1 ? (int)(wn / 2) : (int)wn;
  TORCH_CHECK(mode >= 0 && mode <= 2);
  TORCH_CHECK(x.scalar_type() == at::ScalarType::BFloat16 &&
              w.scalar_type() == at::ScalarType::BFloat16 &&
              y.scalar_type() == at::ScalarType::BFloat16);
  TORCH_CHECK(seg_off.scalar_type() == at::ScalarType::Int &&
              seg_off.numel() == E + 1);
  TORCH_CHECK(N % 128 == 0 && K % 64 == 0 && w.size(2) == K);
  TORCH_CHECK(y.size(0) == T && y.size(1) == N);
  TORCH_CHECK(x.is_contiguous() && w.is_contiguous() && y.is_contiguous());
  if (T == 0) return;
  launch_moe_gemm(ptr<__hip_bfloat16>(y), ptr<__hip_bfloat16>(x),
                  ptr<__hip_bfloat16>(w), ptr<int>(seg_off), E, N, K, T, (int)mode,
                  stream());
}

}  // namespace

void register_par_ops(pybind11::module& m) {
  m.def("stream_add_rms_norm_pair", &stream_add_rms_norm_pair);
  m.def("rope_kv_cache_write", &rope_kv_cache_write);
  m.def("sigmoid_gate_mul", &sigmoid_gate_mul);
  m.def("relu2", &relu2);
  m.def("moe_route", &moe_route);
  m.def("moe_route_sigmoid", &moe_route_sigmoid);
  m.def("moe_combine", &moe_combine);
  m.def("moe_sort", &moe_sort);
  m.def("moe_gemm", &moe_gemm);
}
