// Torch bindings of the `_C_seq` extension: f32 residual-stream ops and the
// short causal convolution with per-sequence state (bindings_rec.cpp adds
// the layer norms, any-shape attention and recurrences).
// Built in-tree by kernels/build.py (hipcc --offload-arch=gfx950).

#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>

#include <hip/hip_bf16.h>

template <typename T>
void launch_gelu_tanh(T*, const T*, long, const T*, long, int, long, hipStream_t);
template <typename T>
void launch_embedding_scaled(float*, const long*, const T*, float, int, int,
                             hipStream_t);
template <typename T>
void launch_rms_norm_stream(T*, const float*, const float*, float, float, int,
                            int, hipStream_t);
template <typename T>
void launch_stream_add(float*, const T*, const T*, float, T*, long, hipStream_t);
template <typename T>
void launch_stream_add_rms_norm(float*, const T*, const float*, float, float,
                                int, int, T*, const float*, float, float,
                                const float*, hipStream_t);
template <typename T>
void launch_softcap(float*, const T*, float, long, hipStream_t);
template <typename T>
void launch_rope_partial(T*, long, long, const long*, const float*, int, int,
                         int, int, int, float, hipStream_t);
template <typename T>
void launch_latent_kv_write(const T*, const float*, float, const long*,
                            const float*, int, T*, const long*, int, int, int,
                            long, int, float, hipStream_t);
template <typename T>
void launch_causal_conv_state(T*, const T*, const float*, T*, const int*,
                              const int*, const int*, int, int, int, int, int,
                              long, const float*, int, hipStream_t);
// layer norms of the stream, attention of any shape, recurrences
// (bindings_rec.cpp)
void register_rec_ops(pybind11::module& m);
// two-norm residual kernel, rotation + cache write, gates, squared relu,
// expert router and combine (bindings_par.cpp)
void register_par_ops(pybind11::module& m);
// token shift, norm + rotation + cache write, chunk-masked attention, the
// differential combination, HGRN2, weighted gated activation (bindings_mix.cpp)
void register_mix_ops(pybind11::module& m);
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

void gelu_tanh(torch::Tensor out, torch::Tensor x,
               c10::optional<torch::Tensor> mul) {
  // x: contiguous of any rank, or a 2-D column slice (rows strided)
  TORCH_CHECK(x.is_cuda() && out.is_contiguous() &&
              (x.is_contiguous() || (x.dim() == 2 && x.stride(1) == 1)));
  TORCH_CHECK(out.scalar_type() == x.scalar_type() && out.numel() == x.numel());
  const int cols = x.size(-1);
  const long x_stride = x.is_contiguous() ? cols : (long)x.stride(0);
  long mul_stride = 0;
  if (mul.has_value()) {
    const auto& m = mul.value();
    TORCH_CHECK(m.dim() == 2 && x.dim() == 2 && m.size(0) == x.size(0) &&
                m.size(1) == cols && m.stride(1) == 1 &&
                m.scalar_type() == x.scalar_type(), "gelu_tanh: bad mul");
    mul_stride = m.stride(0);
  }
  DISPATCH_F32_BF16(x.scalar_type(), {
    launch_gelu_tanh<scalar_t>(
        ptr<scalar_t>(out), ptr<scalar_t>(x), x_stride,
        mul.has_value() ? ptr<scalar_t>(mul.value()) : nullptr, mul_stride,
        cols, x.numel(), stream());
  });
}

void embedding_scaled(torch::Tensor out, torch::Tensor ids, torch::Tensor table,
                      double scale) {
  check_f32(out, "out");
  check_i64(ids, "ids");
  TORCH_CHECK(table.is_cuda() && table.is_contiguous() && table.dim() == 2);
  TORCH_CHECK(out.size(0) == ids.numel() && out.size(1) == table.size(1));
  DISPATCH_F32_BF16(table.scalar_type(), {
    launch_embedding_scaled<scalar_t>(ptr<float>(out), ptr<long>(ids),
                                      ptr<scalar_t>(table), (float)scale,
                                      (int)ids.numel(), (int)table.size(1),
                                      stream());
  });
}

void rms_norm_stream(torch::Tensor out, torch::Tensor x, torch::Tensor weight,
                     double eps, double offset) {
  check_f32(x, "x");
  check_f32(weight, "weight");
  const int width = x.size(-1);
  TORCH_CHECK(out.is_contiguous() && out.numel() == x.numel() &&
              weight.numel() == width);
  const int rows = x.numel() / width;
  DISPATCH_F32_BF16(out.scalar_type(), {
    launch_rms_norm_stream<scalar_t>(ptr<scalar_t>(out), ptr<float>(x),
                                     ptr<float>(weight), (float)eps,
                                     (float)offset, rows, width, stream());
  });
}

void stream_add(torch::Tensor x, torch::Tensor a, c10::optional<torch::Tensor> b,
                double mult, c10::optional<torch::Tensor> cast) {
  check_f32(x, "x");
  TORCH_CHECK(a.is_cuda() && a.is_contiguous() && a.numel() == x.numel());
  if (b.has_value())
    TORCH_CHECK(b.value().is_contiguous() && b.value().numel() == x.numel() &&
                b.value().scalar_type() == a.scalar_type());
  if (cast.has_value())
    TORCH_CHECK(cast.value().is_contiguous() && cast.value().numel() == x.numel() &&
                cast.value().scalar_type() == a.scalar_type());
  DISPATCH_F32_BF16(a.scalar_type(), {
    launch_stream_add<scalar_t>(
        ptr<float>(x), ptr<scalar_t>(a),
        b.has_value() ? ptr<scalar_t>(b.value()) : nullptr, (float)mult,
        cast.has_value() ? ptr<scalar_t>(cast.value()) : nullptr, x.numel(),
        stream());
  });
}

void stream_add_rms_norm(torch::Tensor x, torch::Tensor y, torch::Tensor weight,
                         double eps, double mult,
                         c10::optional<torch::Tensor> next_out,
                         c10::optional<torch::Tensor> next_weight,
                         double next_eps, double next_offset,
                         c10::optional<torch::Tensor> layer_scale) {
  // next_out without next_weight: the updated stream rounded to y's type
  check_f32(x, "x");
  check_f32(weight, "weight");
  const int width = x.size(-1);
  TORCH_CHECK(y.is_cuda() && y.is_contiguous() && y.numel() == x.numel() &&
              weight.numel() == width);
  const int rows = x.numel() / width;
  TORCH_CHECK(next_out.has_value() || !next_weight.has_value());
  if (layer_scale.has_value()) {
    check_f32(layer_scale.value(), "layer_scale");
    TORCH_CHECK(layer_scale.value().numel() == width);
  }
  if (next_weight.has_value()) {
    check_f32(next_weight.value(), "next_weight");
    TORCH_CHECK(next_weight.value().numel() == width);
  }
  if (next_out.has_value()) {
    TORCH_CHECK(next_out.value().is_cuda() && next_out.value().is_contiguous() &&
                next_out.value().numel() == x.numel() &&
                next_out.value().scalar_type() == y.scalar_type());
  }
  DISPATCH_F32_BF16(y.scalar_type(), {
    launch_stream_add_rms_norm<scalar_t>(
        ptr<float>(x), ptr<scalar_t>(y), ptr<float>(weight), (float)eps,
        (float)mult, rows, width,
        next_out.has_value() ? ptr<scalar_t>(next_out.value()) : nullptr,
        next_weight.has_value() ? ptr<float>(next_weight.value()) : nullptr,
        (float)next_eps, (float)next_offset,
        layer_scale.has_value() ? ptr<float>(layer_scale.value()) : nullptr, stream());
  });
}

void softcap(torch::Tensor out, torch::Tensor in, double cap) {
  check_f32(out, "out");
  TORCH_CHECK(in.is_cuda() && in.is_contiguous() && in.numel() == out.numel());
  DISPATCH_F32_BF16(in.scalar_type(), {
    launch_softcap<scalar_t>(ptr<float>(out), ptr<scalar_t>(in), (float)cap,
                             in.numel(), stream());
  });
}

void rope_partial(torch::Tensor x, torch::Tensor positions,
                  torch::Tensor inv_freq, int64_t offset, int64_t rot_dims,
                  bool interleaved, double mag) {
  TORCH_CHECK(x.is_cuda() && x.dim() == 3 && x.stride(2) == 1);
  check_i64(positions, "positions");
  check_f32(inv_freq, "inv_freq");
  const int half = rot_dims / 2;
  TORCH_CHECK(rot_dims % 2 == 0 && inv_freq.numel() >= half &&
              offset >= 0 && offset + rot_dims <= x.size(2) &&
              positions.numel() == x.size(0), "rope_partial: bad shapes");
  if (half == 0) return;
  DISPATCH_F32_BF16(x.scalar_type(), {
    launch_rope_partial<scalar_t>(ptr<scalar_t>(x), x.stride(0), x.stride(1),
                                  ptr<long>(positions), ptr<float>(inv_freq),
                                  (int)x.size(0), (int)x.size(1), (int)offset,
                                  half, interleaved ? 1 : 0, (float)mag,
                                  stream());
  });
}

void latent_kv_write(torch::Tensor dkv, torch::Tensor norm_w, double eps,
                     torch::Tensor positions, torch::Tensor inv_freq,
                     int64_t rot_dims, torch::Tensor cache,
                     torch::Tensor slot_mapping, bool interleaved, double mag) {
  TORCH_CHECK(dkv.is_cuda() && dkv.dim() == 2 && dkv.stride(1) == 1);
  check_f32(norm_w, "norm_w");
  check_f32(inv_freq, "inv_freq");
  check_i64(positions, "positions");
  check_i64(slot_mapping, "slot_mapping");
  const int rank = norm_w.numel();
  const int rot = dkv.size(1) - rank;
  TORCH_CHECK(rot >= 0 && rot_dims % 2 == 0 && rot_dims <= rot &&
              inv_freq.numel() >= rot_dims / 2);
  TORCH_CHECK(cache.is_contiguous() && cache.dim() == 3 &&
              cache.size(2) == dkv.size(1) &&
              cache.scalar_type() == dkv.scalar_type());
  TORCH_CHECK(positions.numel() == dkv.size(0) &&
              slot_mapping.numel() == dkv.size(0));
  DISPATCH_F32_BF16(dkv.scalar_type(), {
    launch_latent_kv_write<scalar_t>(
        ptr<scalar_t>(dkv), ptr<float>(norm_w), (float)eps, ptr<long>(positions),
        ptr<float>(inv_freq), (int)(rot_dims / 2), ptr<scalar_t>(cache),
        ptr<long>(slot_mapping), (int)dkv.size(0), rank, rot,
        (long)dkv.stride(0), interleaved ? 1 : 0, (float)mag, stream());
  });
}

void causal_conv_state(torch::Tensor out, torch::Tensor h, torch::Tensor weight,
                       torch::Tensor state, torch::Tensor loc,
                       torch::Tensor seq_lens, torch::Tensor slots,
                       bool add_input, c10::optional<torch::Tensor> bias,
                       int64_t act) {
  TORCH_CHECK(h.is_cuda() && h.dim() == 2 && h.stride(1) == 1 &&
              out.is_contiguous() && out.scalar_type() == h.scalar_type() &&
              out.numel() == h.numel());
  if (bias.has_value()) {
    check_f32(bias.value(), "bias");
    TORCH_CHECK(bias.value().numel() == h.size(1));
  }
  TORCH_CHECK(act == 0 || act == 1, "act: 0 = none, 1 = silu");
  check_f32(weight, "weight");
  check_i32(loc, "seq_start_loc");
  check_i32(seq_lens, "seq_lens");
  check_i32(slots, "state_slots");
  const int width = h.size(1);
  const int taps = weight.size(1);
  const int nseq = seq_lens.numel();
  TORCH_CHECK(weight.size(0) == width && loc.numel() == nseq + 1 &&
              slots.numel() == nseq && taps >= 1);
  TORCH_CHECK(state.is_contiguous() && state.scalar_type() == h.scalar_type() &&
              state.dim() == 3 && state.size(1) == taps - 1 &&
              (taps == 1 || state.size(2) == width), "conv state shape");
  DISPATCH_F32_BF16(h.scalar_type(), {
    launch_causal_conv_state<scalar_t>(
        ptr<scalar_t>(out), ptr<scalar_t>(h), ptr<float>(weight),
        ptr<scalar_t>(state), ptr<int>(loc), ptr<int>(seq_lens), ptr<int>(slots),
        (int)h.size(0), nseq, width, taps, add_input ? 1 : 0, (long)h.stride(0),
        bias.has_value() ? ptr<float>(bias.value()) : nullptr, (int)act,
        stream());
  });
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("gelu_tanh", &gelu_tanh);
  m.def("embedding_scaled", &embedding_scaled);
  m.def("rms_norm_stream", &rms_norm_stream);
  m.def("stream_add", &stream_add);
  m.def("stream_add_rms_norm", &stream_add_rms_norm);
  m.def("softcap", &softcap);
  m.def("rope_partial", &rope_partial);
  m.def("latent_kv_write", &latent_kv_write);
  m.def("causal_conv_state", &causal_conv_state);
  register_rec_ops(m);
  register_par_ops(m);
  register_mix_ops(m);
}
