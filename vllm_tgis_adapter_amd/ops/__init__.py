"""Custom-op dispatch.

GPU tensors run the hand-written CDNA4 HIP kernels from the in-tree ``_C``
extension (kernels/ — built by ``__graft_entry__.build()`` for gfx950).  CPU
tensors run the plain-PyTorch reference (ops/reference.py), which keeps the
full engine runnable in CPU-only CI like the reference's CPU vLLM build
(SURVEY.md §4).  On a GPU box a missing extension is a hard error — there is
deliberately no silent eager fallback.
"""

from __future__ import annotations

import os

import torch

from . import reference

_C = None
_load_error: str | None = None


def _try_load_native() -> None:
    global _C, _load_error
    if _C is not None:
        return
    try:
        from vllm_tgis_adapter_amd import _C as ext  # in-tree built .so

        _C = ext
    except ImportError as e:
        _load_error = str(e)


_try_load_native()

_FORCE_REFERENCE = os.environ.get("VTA_FORCE_REFERENCE", "0") == "1"


def has_native() -> bool:
    return _C is not None


def native_enabled(t: torch.Tensor) -> bool:
    """True when the HIP path applies to this tensor (device, build, and the
    VTA_FORCE_REFERENCE escape hatch all considered) — non-raising."""
    return t.device.type == "cuda" and not _FORCE_REFERENCE and _C is not None


def _native(t: torch.Tensor) -> bool:
    if t.device.type != "cuda":
        return False
    if _FORCE_REFERENCE:
        return False
    if _C is None:
        raise RuntimeError(
            "vllm_tgis_adapter_amd._C HIP extension is not built but a GPU "
            f"tensor reached a custom op (import error: {_load_error}). "
            "Run `python -c 'import __graft_entry__; __graft_entry__.build()'` "
            "or kernels/build.py first."
        )
    return True


# ---------------------------------------------------------------------------


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    if _native(x):
        out = torch.empty_like(x)
        _C.rms_norm(out, x, weight, eps)
        return out
    return reference.rms_norm(x, weight, eps)


def fused_add_rms_norm(
    x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float
) -> tuple[torch.Tensor, torch.Tensor]:
    """x <- rmsnorm(x + residual); residual <- x + residual (in place on GPU)."""
    if _native(x):
        _C.fused_add_rms_norm(x, residual, weight, eps)
        return x, residual
    return reference.fused_add_rms_norm(x, residual, weight, eps)


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    if x.numel() == 0:
        return x[..., : x.shape[-1] // 2].clone()
    if _native(x):
        d = x.shape[-1] // 2
        out = torch.empty(*x.shape[:-1], d, dtype=x.dtype, device=x.device)
        _C.silu_and_mul(out, x)
        return out
    return reference.silu_and_mul(x)


def rotary_embedding(
    positions: torch.Tensor,
    q: torch.Tensor,
    k: torch.Tensor,
    head_dim: int,
    cos_sin_cache: torch.Tensor,
) -> tuple[torch.Tensor, torch.Tensor]:
    """NeoX rotary; in place on GPU, out-of-place on CPU."""
    if _native(q):
        _C.rotary_embedding(positions, q, k, head_dim, cos_sin_cache)
        return q, k
    return reference.rotary_embedding(positions, q, k, head_dim, cos_sin_cache)


def reshape_and_cache(
    k: torch.Tensor,
    v: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    slot_mapping: torch.Tensor,
) -> None:
    if _native(k):
        _C.reshape_and_cache(k, v, k_cache, v_cache, slot_mapping)
        return
    if k_cache.dtype == torch.uint8:  # fp8 KV: quantize via torch e4m3
        reference.reshape_and_cache(
            k.to(torch.float8_e4m3fn).view(torch.uint8),
            v.to(torch.float8_e4m3fn).view(torch.uint8),
            k_cache, v_cache, slot_mapping)
        return
    reference.reshape_and_cache(k, v, k_cache, v_cache, slot_mapping)


def paged_attention_decode(
    q: torch.Tensor,            # [N, num_heads, head_dim] — one token per seq
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_tables: torch.Tensor,  # [N, max_blocks] int32, device
    seq_lens: torch.Tensor,      # [N] int32, device
    scale: float,
    max_seq_len: int,
    out: torch.Tensor | None = None,
) -> torch.Tensor:
    if _native(q):
        if out is None:
            out = torch.empty_like(q)
        _C.paged_attention_decode(
            out, q, k_cache, v_cache, block_tables, seq_lens, scale
        )
        return out
    n = q.shape[0]
    qsl = torch.arange(n + 1, dtype=torch.int32)
    if k_cache.dtype == torch.uint8:  # fp8 KV: dequantize for the reference
        k_cache = k_cache.view(torch.float8_e4m3fn).to(q.dtype)
        v_cache = v_cache.view(torch.float8_e4m3fn).to(q.dtype)
    r = reference.paged_attention(
        q, k_cache, v_cache, block_tables.cpu(), qsl, seq_lens.cpu(), scale
    )
    if out is not None:
        out.copy_(r)
        return out
    return r


def paged_attention_prefill(
    q: torch.Tensor,               # [T, num_heads, head_dim]
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_tables: torch.Tensor,    # [num_seqs, max_blocks] int32 device
    query_start_loc: torch.Tensor,  # [num_seqs+1] int32 device
    seq_lens: torch.Tensor,         # [num_seqs] int32 device
    scale: float,
    max_query_len: int,
    max_seq_len: int,
) -> torch.Tensor:
    if _native(q):
        out = torch.empty_like(q)
        _C.paged_attention_prefill(
            out, q, k_cache, v_cache, block_tables, query_start_loc, seq_lens,
            scale, max_query_len
        )
        return out
    if k_cache.dtype == torch.uint8:  # fp8 KV: dequantize for the reference
        k_cache = k_cache.view(torch.float8_e4m3fn).to(q.dtype)
        v_cache = v_cache.view(torch.float8_e4m3fn).to(q.dtype)
    return reference.paged_attention(
        q, k_cache, v_cache, block_tables.cpu(), query_start_loc.cpu(),
        seq_lens.cpu(), scale
    )


def linear(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """F.linear with a custom CDNA4 skinny-GEMM path for small decode batches.

    hipBLASLt runs the M<=64 llama decode shapes at 22-43% of the HBM
    roofline (tools/gemm_bench.py); the hand-written MFMA kernel streams the
    weight matrix once with waves splitting K in-workgroup.  Larger M stays
    on hipBLASLt (the in-tree tile kernel only reached parity there —
    VTA_GEMM_MAX_M raises the cutover for experiments).
    """
    max_m = int(os.environ.get("VTA_GEMM_MAX_M", "64"))
    tile_max_m = int(os.environ.get("VTA_GEMM_TILE_MAX_M", "0"))
    if (
        bias is None
        and x.dim() == 2
        and native_enabled(x)
        and x.dtype == torch.bfloat16
        and weight.dtype == torch.bfloat16
        and weight.shape[0] % 128 == 0
        and x.shape[1] % 64 == 0
        and x.is_contiguous()
        and weight.is_contiguous()
    ):
        m = x.shape[0]
        if 1 <= m <= max_m:
            out = torch.empty(
                (m, weight.shape[0]), dtype=x.dtype, device=x.device
            )
            _C.gemm_skinny(out, x, weight)
            return out
        if max_m < m <= tile_max_m:
            out = torch.empty(
                (m, weight.shape[0]), dtype=x.dtype, device=x.device
            )
            _C.gemm_tile(out, x, weight)
            return out
    return torch.nn.functional.linear(x, weight, bias)


def gemm_tile(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """Direct 128x128-tile GEMM path (benchmarks/tests)."""
    assert _native(x)
    out = torch.empty((x.shape[0], weight.shape[0]), dtype=x.dtype, device=x.device)
    _C.gemm_tile(out, x, weight)
    return out


# ---------------------------------------------------------------------------
# Weight-only quantization: RTN into int8 (per-out-channel
# scale) or packed int4 with group-128 scales (the --quantize awq/gptq/
# squeezellm 4-bit surface; offline RTN since checkpoint-specific scales
# don't exist in this environment).
# ---------------------------------------------------------------------------

def quantize_weight(w: torch.Tensor, qbits: int) -> tuple[torch.Tensor, torch.Tensor]:
    """Returns (wq, scales). int8: wq [N,K] int8, scales [N] f32.
    int4: wq [N,K/2] uint8 offset-binary nibbles, scales [N,K/128] f32."""
    assert qbits in (8, 4)
    wf = w.float()
    if qbits == 8:
        scales = wf.abs().amax(dim=1).clamp(min=1e-8) / 127.0
        q = torch.round(wf / scales.unsqueeze(1)).clamp(-127, 127).to(torch.int8)
        return q, scales.contiguous()
    n, k = wf.shape
    assert k % 128 == 0
    g = wf.view(n, k // 128, 128)
    scales = g.abs().amax(dim=2).clamp(min=1e-8) / 7.0
    q = torch.round(g / scales.unsqueeze(2)).clamp(-8, 7).to(torch.int16) + 8
    q = q.view(n, k)
    packed = (q[:, 0::2] | (q[:, 1::2] << 4)).to(torch.uint8)
    return packed.contiguous(), scales.contiguous()


def dequantize_weight(wq: torch.Tensor, scales: torch.Tensor, qbits: int,
                      dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    if qbits == 8:
        return (wq.float() * scales.unsqueeze(1)).to(dtype)
    n = wq.shape[0]
    lo = (wq & 0xF).to(torch.float32) - 8.0
    hi = (wq >> 4).to(torch.float32) - 8.0
    q = torch.stack([lo, hi], dim=2).view(n, -1)  # interleave even/odd k
    k = q.shape[1]
    return (q.view(n, k // 128, 128) * scales.unsqueeze(2)).view(n, k).to(dtype)


def linear_quant(x: torch.Tensor, wq: torch.Tensor, scales: torch.Tensor,
                 qbits: int, bias: torch.Tensor | None = None) -> torch.Tensor:
    """W8A16/W4A16 linear: native dequant-GEMM for decode batches, dequant +
    hipBLASLt above (prefill is compute-bound; the quant win is the weight
    stream at small M)."""
    x2 = x.reshape(-1, x.shape[-1])
    m = x2.shape[0]
    n = wq.shape[0]
    k = x2.shape[1]
    if (
        bias is None
        and _native(x)
        and x.dtype == torch.bfloat16
        and 1 <= m <= 64
        and n % 128 == 0
        and k % 128 == 0
        and x2.is_contiguous()
    ):
        out = torch.empty((m, n), dtype=x.dtype, device=x.device)
        _C.gemm_skinny_q(out, x2, wq, scales, qbits)
        return out.view(*x.shape[:-1], n)
    w = dequantize_weight(wq, scales, qbits, x.dtype)
    return torch.nn.functional.linear(x, w, bias)


def gated_mlp_up(x: torch.Tensor, w13: torch.Tensor) -> torch.Tensor | None:
    """Fused silu(x@Wg^T) * (x@Wu^T) for merged [gate; up] weights.

    Returns None when the fused CDNA4 path doesn't apply (caller falls back
    to linear + silu_and_mul).
    """
    max_m = int(os.environ.get("VTA_GEMM_MAX_M", "64"))
    if (
        x.dim() == 2
        and 1 <= x.shape[0] <= max_m
        and x.dtype == torch.bfloat16
        and w13.dtype == torch.bfloat16
        and w13.shape[0] % 256 == 0
        and x.shape[1] % 64 == 0
        and x.is_contiguous()
        and w13.is_contiguous()
        and _native(x)
    ):
        inter = w13.shape[0] // 2
        out = torch.empty((x.shape[0], inter), dtype=x.dtype, device=x.device)
        _C.gemm_skinny_gated(out, x, w13)
        return out
    return None


def lora_bgmv(
    out: torch.Tensor,      # [T, out_w] updated in place
    x: torch.Tensor,        # [T, K]
    a_stack: torch.Tensor,  # [L, R, K]
    b_stack: torch.Tensor,  # [L, N, R]
    slots: torch.Tensor,    # [T] int32, -1 = no adapter
    scales: torch.Tensor,   # [L] float32
    off: int,
) -> None:
    """Batched LoRA delta for a mixed-adapter batch (GPU only)."""
    assert _native(x), "lora_bgmv is the GPU path; CPU uses the torch loop"
    tmp = torch.empty(
        (x.shape[0], a_stack.shape[1]), dtype=torch.float32, device=x.device
    )
    _C.lora_bgmv(out, x, a_stack, b_stack, tmp, slots, scales, off)


def sample_argmax(
    out: torch.Tensor,     # [N] int64
    logits: torch.Tensor,  # [N, V]
    temps: torch.Tensor,   # [N] float32, 0 = greedy
    noise: torch.Tensor | None,  # [N, V] float32 Exp(1) draws for temp>0 rows
) -> None:
    """Fused temperature + exponential-race sampling / greedy argmax (E7)."""
    assert _native(logits), "sample_argmax is the GPU path"
    _C.sample_argmax(out, logits, temps, noise)


def logsoftmax_topk_usable(logits: torch.Tensor) -> bool:
    # V >= 2048 guarantees every lane feeds both accumulator pairs
    return (native_enabled(logits) and logits.dtype == torch.bfloat16
            and logits.shape[1] % 8 == 0 and logits.shape[1] >= 2048)


def logsoftmax_topk(
    logits: torch.Tensor,  # [N, V] bf16 (contiguous)
    chosen: torch.Tensor,  # [N] int64 sampled/actual token per row
    k: int,
):
    """Fused log-softmax + top-K + chosen-token logprob/rank in one HBM
    pass (E8 wire details).  Returns (topv f32 [N,K], topi i32 [N,K],
    chosen_lp f32 [N], ranks i32 [N]); launch only, no host sync."""
    assert logsoftmax_topk_usable(logits), "logsoftmax_topk is the GPU path"
    n = logits.shape[0]
    dev = logits.device
    topv = torch.empty((n, k), dtype=torch.float32, device=dev)
    topi = torch.empty((n, k), dtype=torch.int32, device=dev)
    chosen_lp = torch.empty((n,), dtype=torch.float32, device=dev)
    ranks = torch.empty((n,), dtype=torch.int32, device=dev)
    _C.logsoftmax_topk(topv, topi, chosen_lp, ranks,
                       logits.contiguous(), chosen.contiguous())
    return topv, topi, chosen_lp, ranks


def moe_gemm(
    x: torch.Tensor,        # [T, K] rows sorted by expert
    w: torch.Tensor,        # [E, 2N, K] (gated) or [E, N, K]
    seg_off: torch.Tensor,  # [E+1] int32 device row offsets
    gated: bool,
    act: str | None = None,
) -> torch.Tensor:
    """Grouped GEMM over expert segments (E16); gated fuses SiLU(g)*u; a plain
    product may be followed by ``act`` ("relu2": the squared relu).  Rows past
    the last segment are left unwritten."""
    if act not in (None, "relu2") or (gated and act):
        raise ValueError(f"unknown activation {act!r}")
    n = w.shape[1] // 2 if gated else w.shape[1]
    if x.device.type != "cuda" or _FORCE_REFERENCE:
        return reference.moe_gemm(x, w, seg_off.cpu(), gated, act)
    ext = _C if _C is not None else (_S if _native_seq(x) else None)
    out = torch.empty((x.shape[0], n), dtype=x.dtype, device=x.device)
    ext.moe_gemm(out, x, w, seg_off, 1 if gated else (2 if act == "relu2" else 0))
    return out


def moe_gemm_usable(x: torch.Tensor, hidden: int, inter: int) -> bool:
    return (
        native_enabled(x)
        and x.dtype == torch.bfloat16
        and inter % 128 == 0
        and hidden % 128 == 0
        and hidden % 64 == 0
    )


def topk_softmax(gate_logits: torch.Tensor, top_k: int):
    # Router math is tiny; torch ops are fine on both devices for now.
    return reference.topk_softmax(gate_logits, top_k)


make_cos_sin_cache = reference.make_cos_sin_cache


# ---------------------------------------------------------------------------
# `_C_seq`: f32 residual-stream ops, short causal convolution with
# per-sequence state (further down: layer norms, any-shape attention,
# recurrences); `_C_lat`: windowed latent attention with sinks.  Separate
# extensions so a model that needs only these compiles only these.
# ---------------------------------------------------------------------------

_S = None
_seq_load_error: str | None = None


def _try_load_seq() -> None:
    global _S, _seq_load_error
    if _S is not None:
        return
    try:
        from vllm_tgis_adapter_amd import _C_seq as ext

        _S = ext
    except ImportError as e:
        _seq_load_error = str(e)


_try_load_seq()


_L = None          # `_C_lat`: latent attention
_A = None          # `_C_attn`: paged attention alone (when `_C` is not built)
_lat_load_error: str | None = None


def _try_load_lat() -> None:
    global _L, _lat_load_error
    if _L is not None:
        return
    try:
        from vllm_tgis_adapter_amd import _C_lat as ext

        _L = ext
    except ImportError as e:
        _lat_load_error = str(e)


def _try_load_attn() -> None:
    global _A
    if _A is not None or _C is not None:
        return
    try:
        from vllm_tgis_adapter_amd import _C_attn as ext

        _A = ext
    except ImportError:
        pass


_try_load_lat()
_try_load_attn()


def _native_lat(t: torch.Tensor) -> bool:
    if t.device.type != "cuda" or _FORCE_REFERENCE:
        return False
    if _L is None:
        _try_load_lat()
    if _L is None:
        raise RuntimeError(
            "vllm_tgis_adapter_amd._C_lat HIP extension is not built but a GPU "
            f"tensor reached one of its ops (import error: {_lat_load_error}). "
            "Run `python kernels/build.py --only=_C_lat` first."
        )
    return True


def _attn_ext():
    """The extension that holds the llama-class paged attention kernels: all
    of ``_C`` when it is built, else the attention-only ``_C_attn``."""
    return _C if _C is not None else _A


def reload_native() -> None:
    """Load extensions that were built after this module was imported."""
    _try_load_native()
    _try_load_seq()
    _try_load_lat()
    _try_load_attn()


def has_native_seq() -> bool:
    _try_load_seq()
    return _S is not None


def _native_seq(t: torch.Tensor) -> bool:
    if t.device.type != "cuda" or _FORCE_REFERENCE:
        return False
    if _S is None:
        _try_load_seq()
    if _S is None:
        raise RuntimeError(
            "vllm_tgis_adapter_amd._C_seq HIP extension is not built but a GPU "
            f"tensor reached one of its ops (import error: {_seq_load_error}). "
            "Run `python kernels/build.py --only=_C_seq` first."
        )
    return True


def gelu_tanh(x: torch.Tensor, mul: torch.Tensor | None = None) -> torch.Tensor:
    """tanh-form GELU, optionally times ``mul``; x and mul may be column
    slices of a wider matrix (strided rows)."""
    if x.numel() and _native_seq(x):
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        _S.gelu_tanh(out, x, mul)
        return out
    return reference.gelu_tanh(x, mul)


def embedding_scaled(ids: torch.Tensor, table: torch.Tensor, scale: float) -> torch.Tensor:
    """f32 rows table[ids] * scale — the start of an f32 residual stream."""
    if ids.numel() and _native_seq(table):
        out = torch.empty((ids.shape[0], table.shape[1]), dtype=torch.float32,
                          device=table.device)
        _S.embedding_scaled(out, ids, table, float(scale))
        return out
    return reference.embedding_scaled(ids, table, scale)


def rms_norm_stream(x: torch.Tensor, weight: torch.Tensor, eps: float,
                    weight_offset: float, out_dtype: torch.dtype) -> torch.Tensor:
    """RMS norm of an f32 stream, weight applied as (weight_offset + w)."""
    if x.numel() and _native_seq(x):
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        _S.rms_norm_stream(out, x, weight, float(eps), float(weight_offset))
        return out
    return reference.rms_norm_stream(x, weight, eps, weight_offset, out_dtype)


def stream_add(x: torch.Tensor, a: torch.Tensor, b: torch.Tensor | None,
               mult: float, cast_dtype: torch.dtype | None = None):
    """x (f32, in place) += mult * (a + b); optionally also returns the new x
    rounded to ``cast_dtype`` for the next projection."""
    if x.numel() and _native_seq(x):
        cast = (torch.empty(x.shape, dtype=cast_dtype, device=x.device)
                if cast_dtype is not None else None)
        _S.stream_add(x, a, b, float(mult), cast)
        return cast
    return reference.stream_add(x, a, b, mult, cast_dtype)


def stream_add_rms_norm(x: torch.Tensor, y: torch.Tensor, weight: torch.Tensor,
                        eps: float, mult: float, next_norm=None,
                        layer_scale: torch.Tensor | None = None,
                        cast_dtype: torch.dtype | None = None):
    """x (f32, in place) += mult * y / rms(y) * weight (* layer_scale [W] f32).

    ``next_norm`` = (weight, eps, weight_offset, dtype) fuses the following
    norm of the updated stream into the same pass and returns its output;
    ``cast_dtype`` instead returns the updated stream rounded to that dtype
    (for a sublayer that reads the stream itself)."""
    if next_norm is not None and cast_dtype is not None:
        raise ValueError("either the next norm or a cast of the stream, not both")
    if x.numel() and _native_seq(x):
        if next_norm is None:
            out = (torch.empty(x.shape, dtype=cast_dtype, device=x.device)
                   if cast_dtype is not None else None)
            _S.stream_add_rms_norm(x, y, weight, float(eps), float(mult),
                                   out, None, 0.0, 0.0, layer_scale)
            return out
        nw, neps, noff, ndtype = next_norm
        out = torch.empty(x.shape, dtype=ndtype, device=x.device)
        _S.stream_add_rms_norm(x, y, weight, float(eps), float(mult), out, nw,
                               float(neps), float(noff), layer_scale)
        return out
    reference.stream_add_rms_norm(x, y, weight, eps, mult, layer_scale)
    if next_norm is None:
        return x.to(cast_dtype) if cast_dtype is not None else None
    nw, neps, noff, ndtype = next_norm
    return reference.rms_norm_stream(x, nw, neps, noff, ndtype)


def softcap(logits: torch.Tensor, cap: float) -> torch.Tensor:
    """f32 cap * tanh(logits / cap)."""
    if logits.numel() and _native_seq(logits):
        out = torch.empty(logits.shape, dtype=torch.float32, device=logits.device)
        _S.softcap(out, logits.contiguous(), float(cap))
        return out
    return reference.softcap(logits, cap)


def causal_conv_state(h, weight, state, seq_start_loc, seq_lens, state_slots,
                      add_input: bool = True, bias: torch.Tensor | None = None,
                      act: str | None = None) -> torch.Tensor:
    """Depthwise causal convolution over each sequence's new rows with the
    last taps-1 inputs carried in ``state[slot]`` (advanced in place).  ``h``
    may be a column slice of a wider matrix; ``bias`` [W] f32 and ``act``
    ("silu") are applied to the result."""
    if act not in (None, "silu"):
        raise ValueError(f"unknown activation {act!r}")
    if h.numel() and _native_seq(h):
        out = torch.empty(h.shape, dtype=h.dtype, device=h.device)
        _S.causal_conv_state(out, h, weight, state, seq_start_loc, seq_lens,
                             state_slots, bool(add_input), bias,
                             1 if act == "silu" else 0)
        return out
    return reference.causal_conv_state(
        h, weight, state, seq_start_loc.cpu(), seq_lens.cpu(), state_slots.cpu(),
        add_input, bias, act)


def rope_partial(x: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor,
                 offset: int, rot_dims: int, interleaved: bool = False,
                 mag: float = 1.0) -> None:
    """In place rotation of dims [offset, offset+rot_dims) of every head of
    x [T, H, D]: dim i paired with i + rot_dims/2, or (``interleaved``) dim 2i
    with 2i+1; f32 angles position * inv_freq[i], cos and sin times ``mag``."""
    if x.numel() and _native_seq(x):
        _S.rope_partial(x, positions, inv_freq, int(offset), int(rot_dims),
                        bool(interleaved), float(mag))
        return
    reference.rope_partial(x, positions, inv_freq, offset, rot_dims, interleaved, mag)


def latent_kv_write(dkv, norm_weight, eps, positions, inv_freq, rot_dims,
                    cache, slot_mapping, interleaved: bool = False,
                    mag: float = 1.0) -> None:
    """RMS-norm the latent part, rotate the shared key part, store the row in
    the paged latent cache.  ``dkv`` may be a column slice of a wider matrix."""
    if dkv.numel() and _native_seq(dkv):
        _S.latent_kv_write(dkv, norm_weight, float(eps), positions, inv_freq,
                           int(rot_dims), cache, slot_mapping, bool(interleaved),
                           float(mag))
        return
    reference.latent_kv_write(dkv, norm_weight, eps, positions, inv_freq,
                              rot_dims, cache, slot_mapping, interleaved, mag)


def latent_attention_prefill(q_lat, q_rot, cache, block_tables, query_start_loc,
                             seq_lens, scale, window, sinks, max_query_len,
                             out: torch.Tensor, general: bool = False,
                             two_term: bool = False) -> torch.Tensor:
    """Windowed multi-query attention with sinks over the paged latent cache
    for query chunks (the tail rows of each sequence).  bf16 shapes on the
    MFMA kernel's list run there unless ``general`` asks for the any-shape
    kernel (f32 always does).  ``two_term``: on the MFMA kernel the
    probabilities enter the value product as two bf16 terms (rounded value +
    rounded remainder) instead of one."""
    if q_lat.numel() and _native_lat(q_lat):
        _L.latent_attention_prefill(out, q_lat, q_rot, cache, block_tables,
                                    query_start_loc, seq_lens, float(scale),
                                    int(window), sinks, int(max_query_len), bool(general),
                                    bool(two_term))
        return out
    out.copy_(reference.latent_attention(
        q_lat, q_rot, cache, block_tables.cpu(), query_start_loc.cpu(),
        seq_lens.cpu(), scale, window, sinks))
    return out


def latent_attention_decode(q_lat, q_rot, cache, block_tables, seq_lens, scale,
                            window, sinks, out: torch.Tensor,
                            general: bool = False, two_term: bool = False) -> torch.Tensor:
    """Same attention for one new query per sequence."""
    if q_lat.numel() and _native_lat(q_lat):
        _L.latent_attention_decode(out, q_lat, q_rot, cache, block_tables,
                                   seq_lens, float(scale), int(window), sinks,
                                   bool(general), bool(two_term))
        return out
    n = q_lat.shape[0]
    qsl = torch.arange(n + 1, dtype=torch.int32)
    out.copy_(reference.latent_attention(
        q_lat, q_rot, cache, block_tables.cpu(), qsl, seq_lens.cpu(), scale,
        window, sinks))
    return out


# ---------------------------------------------------------------------------
# Layer norm of the f32 stream, grouped-query softmax attention with per-head
# query/key norm (any query/key and value size, f32 or bf16), recurrent mixers
# with per-sequence f32 state.  Same extension as the stream ops.
# ---------------------------------------------------------------------------


def layer_norm_stream(x: torch.Tensor, weight: torch.Tensor, eps: float,
                      out_dtype: torch.dtype) -> torch.Tensor:
    """Bias-free layer norm of an f32 stream into the compute dtype."""
    if x.numel() and _native_seq(x):
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        _S.layer_norm_stream(out, x, weight, float(eps))
        return out
    return reference.layer_norm_stream(x, weight, eps, out_dtype)


def stream_add_layer_norm(x: torch.Tensor, a: torch.Tensor, b: torch.Tensor | None,
                          scale_a: float, scale_b: float, weight: torch.Tensor,
                          layer_scale: torch.Tensor | None, eps: float,
                          next_norm=None):
    """x (f32, in place) += LN(scale_a * a + scale_b * b) * weight * layer_scale.

    ``next_norm`` = (weight, eps, dtype): the layer norm that reads the updated
    stream next is computed in the same pass and returned."""
    if x.numel() and _native_seq(x):
        out = None
        nw, neps = None, 0.0
        if next_norm is not None:
            nw, neps, ndtype = next_norm
            out = torch.empty(x.shape, dtype=ndtype, device=x.device)
        _S.stream_add_layer_norm(x, a, b, float(scale_a), float(scale_b), weight,
                                 layer_scale, float(eps), out, nw, float(neps))
        return out
    reference.stream_add_layer_norm(x, a, b, scale_a, scale_b, weight, layer_scale, eps)
    if next_norm is None:
        return None
    nw, neps, ndtype = next_norm
    return reference.layer_norm_stream(x, nw, neps, ndtype)


def stream_add_vec(x: torch.Tensor, other: torch.Tensor | None, vec: torch.Tensor) -> None:
    """x (f32, in place) += other + vec, vec [width] broadcast over rows."""
    if x.numel() and _native_seq(x):
        _S.stream_add_vec(x, other, vec)
        return
    reference.stream_add_vec(x, other, vec)


def qk_norm_cache_write(q, k, v, q_weight, k_weight, eps, positions, temp_coef,
                        temp_every, k_cache, v_cache, slot_mapping) -> torch.Tensor:
    """Per-head RMS norm of q [T, H, dim] and k [T, G, dim] (views into a merged
    projection are fine), position-dependent query temperature, normed keys and
    v [T, G, vdim] stored in the paged cache.  Returns contiguous queries."""
    if q.numel() and _native_seq(q):
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
        _S.qk_norm_cache_write(out, q, k, v, q_weight, k_weight, float(eps),
                               positions, float(temp_coef), int(temp_every),
                               k_cache, v_cache, slot_mapping)
        return out
    return reference.qk_norm_cache_write(q, k, v, q_weight, k_weight, eps, positions,
                                         temp_coef, temp_every, k_cache, v_cache,
                                         slot_mapping)


def _matrix_core_attention_fits(q: torch.Tensor, k_cache: torch.Tensor,
                                v_cache: torch.Tensor) -> bool:
    """The llama-class MFMA kernels of ``_C`` take bf16, equal query/key and
    value sizes of 64 or 128 and up to 8 query heads per key head."""
    if _attn_ext() is None or _FORCE_REFERENCE or q.dtype != torch.bfloat16:
        return False
    d = q.shape[-1]
    group = q.shape[1] // k_cache.shape[2]
    return (d in (64, 128) and v_cache.shape[-1] == d and 1 <= group <= 8
            and q.shape[1] == group * k_cache.shape[2])


def _windowed_matrix_core_fits(q: torch.Tensor, k_cache: torch.Tensor,
                               v_cache: torch.Tensor, single: bool) -> bool:
    """The window + sink variants of the MFMA kernels take bf16, equal key and
    value size of 128 (single queries: also 64), up to 8 query heads per key
    head."""
    if _attn_ext() is None or _FORCE_REFERENCE or q.dtype != torch.bfloat16:
        return False
    d = q.shape[-1]
    group = q.shape[1] // k_cache.shape[2]
    return (d in ((64, 128) if single else (128,)) and v_cache.shape[-1] == d
            and 1 <= group <= 8 and q.shape[1] == group * k_cache.shape[2]
            and q.is_contiguous())


def windowed_attention_uses_matrix_cores(dtype: torch.dtype, heads: int, kv_heads: int,
                                         dim: int, vdim: int) -> bool:
    """Shape test of the above without tensors (which extensions a model needs)."""
    return (dtype == torch.bfloat16 and dim == vdim and dim in (64, 128)
            and heads % kv_heads == 0 and 1 <= heads // kv_heads <= 8)


def attention_uses_matrix_cores(dtype: torch.dtype, heads: int, kv_heads: int,
                                dim: int, vdim: int) -> bool:
    """Shape test of the above without tensors (which extensions a model needs)."""
    return (dtype == torch.bfloat16 and dim == vdim and dim in (64, 128)
            and heads % kv_heads == 0 and 1 <= heads // kv_heads <= 8)


def gqa_attention_prefill(q, k_cache, v_cache, block_tables, query_start_loc,
                          seq_lens, scale, max_query_len, out: torch.Tensor,
                          window: int = 0, sink: float | None = None) -> torch.Tensor:
    """Causal grouped-query softmax attention of query chunks (the tail rows
    of each sequence) over the paged cache; q [T, H, dim], out [T, H, vdim].
    ``window`` > 0: position i sees j with 0 <= i - j < window.  ``sink``: the
    softmax denominator also holds exp(sink), a key without a value.
    bf16 shapes the MFMA kernels take run there, everything else (f32, other
    sizes, value size unlike the key size) on the any-shape kernel."""
    if q.numel() and _native_seq(q):
        if window > 0 or sink is not None:
            if _windowed_matrix_core_fits(q, k_cache, v_cache, single=False):
                dst = out if out.is_contiguous() else torch.empty_like(q)
                _attn_ext().windowed_attention_prefill(
                    dst, q, k_cache, v_cache, block_tables, query_start_loc, seq_lens,
                    float(scale), int(max_query_len), int(window), sink is not None,
                    float(sink or 0.0))
                if dst is not out:
                    out.copy_(dst)
                return out
            _S.paged_attention_any(out, q, k_cache, v_cache, block_tables,
                                   query_start_loc, seq_lens, float(scale),
                                   int(max_query_len), int(window),
                                   sink is not None, float(sink or 0.0))
            return out
        if _matrix_core_attention_fits(q, k_cache, v_cache):
            dst = out if out.is_contiguous() else torch.empty_like(q)
            _attn_ext().paged_attention_prefill(dst, q, k_cache, v_cache, block_tables,
                                       query_start_loc, seq_lens, float(scale),
                                       int(max_query_len))
            if dst is not out:
                out.copy_(dst)
            return out
        _S.paged_attention_any(out, q, k_cache, v_cache, block_tables,
                               query_start_loc, seq_lens, float(scale),
                               int(max_query_len), 0, False, 0.0)
        return out
    out.copy_(reference.paged_attention(
        q, k_cache, v_cache, block_tables.cpu(), query_start_loc.cpu(),
        seq_lens.cpu(), scale, window, sink))
    return out


def gqa_attention_decode(q, k_cache, v_cache, block_tables, seq_lens, scale,
                         out: torch.Tensor, window: int = 0,
                         sink: float | None = None) -> torch.Tensor:
    """Same attention for one new query per sequence (seq_len 0 = padding row,
    zeros)."""
    if q.numel() and _native_seq(q):
        if window > 0 or sink is not None:
            if _windowed_matrix_core_fits(q, k_cache, v_cache, single=True):
                dst = out if out.is_contiguous() else torch.empty_like(q)
                _attn_ext().windowed_attention_decode(
                    dst, q, k_cache, v_cache, block_tables, seq_lens, float(scale),
                    int(window), sink is not None, float(sink or 0.0))
                if dst is not out:
                    out.copy_(dst)
                return out
            _S.paged_attention_any(out, q, k_cache, v_cache, block_tables, None,
                                   seq_lens, float(scale), 1, int(window),
                                   sink is not None, float(sink or 0.0))
            return out
        if _matrix_core_attention_fits(q, k_cache, v_cache):
            if out.is_contiguous():
                _attn_ext().paged_attention_decode(out, q, k_cache, v_cache,
                                                   block_tables, seq_lens, float(scale))
            else:
                tmp = torch.empty_like(q)
                _attn_ext().paged_attention_decode(tmp, q, k_cache, v_cache,
                                                   block_tables, seq_lens, float(scale))
                out.copy_(tmp)
            return out
        _S.paged_attention_any(out, q, k_cache, v_cache, block_tables, None,
                               seq_lens, float(scale), 1, 0, False, 0.0)
        return out
    n = q.shape[0]
    qsl = torch.arange(n + 1, dtype=torch.int32)
    out.copy_(reference.paged_attention(
        q, k_cache, v_cache, block_tables.cpu(), qsl, seq_lens.cpu(), scale,
        window, sink))
    return out


def ssd_scan(xbc, dt, dt_bias, a_log, d_skip, state, seq_start_loc, seq_lens,
             state_slots, heads: int, vdim: int, nstate: int, groups: int) -> torch.Tensor:
    """State-space-duality recurrence over each sequence's new rows with the
    f32 state [slots, H, vdim, N] advanced in place; returns y [T, H*vdim] f32."""
    if xbc.numel() and _native_seq(xbc):
        y = torch.empty((xbc.shape[0], heads * vdim), dtype=torch.float32,
                        device=xbc.device)
        _S.ssd_scan(y, xbc, dt, dt_bias, a_log, d_skip, state, seq_start_loc,
                    seq_lens, state_slots, int(heads), int(vdim), int(nstate),
                    int(groups))
        return y
    return reference.ssd_scan(xbc, dt, dt_bias, a_log, d_skip, state,
                              seq_start_loc.cpu(), seq_lens.cpu(), state_slots.cpu(),
                              heads, vdim, nstate, groups)


def gated_group_norm(y, gate, weight, groups: int, eps: float, gate_first: bool,
                     out_dtype: torch.dtype) -> torch.Tensor:
    """RMS norm of y [T, C] (f32) in ``groups`` equal parts, times weight, with
    a gate [T, C]: silu(gate) multiplied in before the norm (gate_first) or
    sigmoid(gate) after it."""
    if y.numel() and _native_seq(y):
        out = torch.empty(y.shape, dtype=out_dtype, device=y.device)
        _S.gated_group_norm(out, y, gate, weight, int(groups), float(eps),
                            bool(gate_first))
        return out
    return reference.gated_group_norm(y, gate, weight, groups, eps, gate_first, out_dtype)


def rglru_scan(u, r_pre, i_pre, r_bias, i_bias, lam, gate_c, y_branch, state,
               seq_start_loc, seq_lens, state_slots) -> torch.Tensor:
    """Real-gated linear recurrent unit over each sequence's new rows (f32
    state [slots, W] advanced in place), times the other branch."""
    if u.numel() and _native_seq(u):
        out = torch.empty(u.shape, dtype=u.dtype, device=u.device)
        _S.rglru_scan(out, u, r_pre, i_pre, r_bias, i_bias, lam, float(gate_c),
                      y_branch, state, seq_start_loc, seq_lens, state_slots)
        return out
    return reference.rglru_scan(u, r_pre, i_pre, r_bias, i_bias, lam, gate_c,
                                y_branch, state, seq_start_loc.cpu(), seq_lens.cpu(),
                                state_slots.cpu())


def mlstm_scan(q, k, v, i_pre, f_pre, i_bias, f_bias, cap, q_scale, s_state,
               n_state, m_state, seq_start_loc, seq_lens, state_slots) -> torch.Tensor:
    """mLSTM matrix-memory recurrence over each sequence's new rows (f32 state
    S, n, m advanced in place); returns o [T, H*vdim] f32."""
    if q.numel() and _native_seq(q):
        o = torch.empty((q.shape[0], q.shape[1] * v.shape[-1]), dtype=torch.float32,
                        device=q.device)
        _S.mlstm_scan(o, q, k, v, i_pre, f_pre, i_bias, f_bias, float(cap),
                      float(q_scale), s_state, n_state, m_state, seq_start_loc,
                      seq_lens, state_slots)
        return o
    return reference.mlstm_scan(q, k, v, i_pre, f_pre, i_bias, f_bias, cap, q_scale,
                                s_state, n_state, m_state, seq_start_loc.cpu(),
                                seq_lens.cpu(), state_slots.cpu())


# ---------------------------------------------------------------------------
# Two-norm parallel layers, rotated grouped-query attention whose cache is
# written by one op, output gates, squared-relu feed-forwards, routed experts
# with identity experts.  Same extension as the stream ops.
# ---------------------------------------------------------------------------


def stream_add_rms_norm_pair(x: torch.Tensor, a: torch.Tensor | None,
                             b: torch.Tensor | None, w1: torch.Tensor | None,
                             w2: torch.Tensor | None, eps: float,
                             out_dtype: torch.dtype,
                             row_scale: torch.Tensor | None = None,
                             c: torch.Tensor | None = None):
    """x (f32, in place) += a + b + row_scale[:, None] * c (each optional;
    nothing is added when ``a`` is None), then the two RMS norms that read the
    updated stream next, which share one statistic: x / sqrt(mean(x^2) + eps)
    times w1 and times w2.  Returns (h1, h2), None where the weight is None."""
    if x.numel() and _native_seq(x):
        h1 = torch.empty(x.shape, dtype=out_dtype, device=x.device) if w1 is not None else None
        h2 = torch.empty(x.shape, dtype=out_dtype, device=x.device) if w2 is not None else None
        _S.stream_add_rms_norm_pair(x, a, b, row_scale, c, w1, w2, float(eps), h1, h2)
        return h1, h2
    return reference.stream_add_rms_norm_pair(x, a, b, row_scale, c, w1, w2, eps, out_dtype)


def rope_kv_cache_write(q, k, v, positions, inv_freq, rot_dims: int, interleaved: bool,
                        mag: float, k_cache, v_cache, slot_mapping) -> torch.Tensor:
    """Rotate the first ``rot_dims`` dims of every head of q [T, H, dim] and
    k [T, G, dim] (f32 angles position * inv_freq[i], cos and sin times
    ``mag``), store rotated keys and v [T, G, vdim] as given in the paged cache.
    q, k, v may be views into a merged projection (v may alias k: the values
    are then the unrotated keys).  Returns contiguous rotated queries."""
    if q.numel() and _native_seq(q):
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
        _S.rope_kv_cache_write(out, q, k, v, positions, inv_freq, int(rot_dims),
                               bool(interleaved), float(mag), k_cache, v_cache,
                               slot_mapping)
        return out
    return reference.rope_kv_cache_write(q, k, v, positions, inv_freq, rot_dims,
                                         interleaved, mag, k_cache, v_cache, slot_mapping)


def sigmoid_gate_mul(o: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
    """o [T, H, D] (any head / row strides) times sigmoid(gate) with gate
    [T, H, D] (elementwise) or [T, H] (one per head), f32 sigmoid; returns
    contiguous [T, H * D]."""
    if o.numel() and _native_seq(o):
        t, h, d = o.shape
        out = torch.empty((t, h * d), dtype=o.dtype, device=o.device)
        _S.sigmoid_gate_mul(out, o, gate)
        return out
    return reference.sigmoid_gate_mul(o, gate)


def relu2(x: torch.Tensor, bias: torch.Tensor | None = None,
          col_scale: torch.Tensor | None = None) -> torch.Tensor:
    """relu(x + bias)^2; with ``col_scale`` [T, E] f32 also times
    col_scale[t, column // (columns / E)]."""
    if x.numel() and _native_seq(x):
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        _S.relu2(out, x, bias, col_scale)
        return out
    return reference.relu2(x, bias, col_scale)


def moe_route(logits: torch.Tensor, correction: torch.Tensor, top: int, num_real: int):
    """Softmax router with a choice correction and identity experts; see
    reference.moe_route.  Returns (dense [T, num_real] f32, identity [T] f32,
    ids [T, top] int32, weights [T, top] f32)."""
    if logits.numel() and _native_seq(logits):
        t, n = logits.shape
        dev = logits.device
        dense = torch.empty((t, num_real), dtype=torch.float32, device=dev)
        ident = torch.empty((t,), dtype=torch.float32, device=dev)
        ids = torch.empty((t, top), dtype=torch.int32, device=dev)
        w = torch.empty((t, top), dtype=torch.float32, device=dev)
        _S.moe_route(dense, ident, ids, w, logits, correction, int(num_real))
        return dense, ident, ids, w
    return reference.moe_route(logits, correction, top, num_real)


def moe_combine(ye: torch.Tensor, pos: torch.Tensor, ids: torch.Tensor,
                weights: torch.Tensor, num_real: int) -> torch.Tensor:
    """Weighted sum of each token's real-expert outputs, gathered from the
    expert-sorted rows ``ye`` through ``pos`` [T, top]; no atomics."""
    if ye.numel() and _native_seq(ye):
        out = torch.empty((pos.shape[0], ye.shape[1]), dtype=ye.dtype, device=ye.device)
        _S.moe_combine(out, ye, pos, ids, weights, int(num_real))
        return out
    return reference.moe_combine(ye, pos, ids, weights, num_real)


def moe_sort(ids: torch.Tensor, num_real: int, h: torch.Tensor,
             row_scale: torch.Tensor | None = None):
    """Group the token-expert pairs ids [T, top] by expert.  Returns (xs
    [T * top, W]: h's rows gathered so that expert e's pairs fill rows seg[e] ..
    seg[e+1], pos [T, top] int32: the row of each pair (0 for identity experts,
    ids >= num_real, which get no row), seg [num_real + 1] int32).  Rows past
    seg[-1] are left unwritten.  The order of the pairs inside a segment is
    not specified.  ``row_scale`` [T, top] f32: pair (t, k)'s gathered row is
    h[t] times row_scale[t, k], rounded once."""
    if h.numel() and _native_seq(h):
        t, top = ids.shape
        dev = h.device
        xs = torch.empty((t * top, h.shape[1]), dtype=h.dtype, device=dev)
        pos = torch.empty((t, top), dtype=torch.int32, device=dev)
        seg = torch.empty((num_real + 1,), dtype=torch.int32, device=dev)
        scratch = torch.zeros((2 * num_real,), dtype=torch.int32, device=dev)
        _S.moe_sort(xs, pos, seg, scratch, h, ids, int(num_real), row_scale)
        return xs, pos, seg
    return reference.moe_sort(ids, num_real, h, row_scale)


# ---------------------------------------------------------------------------
# Token shift with per-sequence state, query/key norm + rotation + cache
# write, chunk-masked attention with shared value heads and the differential
# combination of two maps, the HGRN2 recurrence, sigmoid routing and gated
# experts fed weighted inputs.  Same extension as the stream ops.
# ---------------------------------------------------------------------------


def token_shift_state(x: torch.Tensor, weight: torch.Tensor, state: torch.Tensor,
                      seq_start_loc, seq_lens, state_slots,
                      out_dtype: torch.dtype) -> torch.Tensor:
    """x_t + (x_(t-1) - x_t) * weight over each sequence's new rows of the f32
    stream, in the compute dtype; the row before a portion comes from
    ``state[slot]`` (f32, zero before position 0), which then takes the
    portion's last row."""
    if x.numel() and _native_seq(x):
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        _S.token_shift_state(out, x, weight, state, seq_start_loc, seq_lens, state_slots)
        return out
    return reference.token_shift_state(x, weight, state, seq_start_loc.cpu(),
                                       seq_lens.cpu(), state_slots.cpu(), out_dtype)


def qk_norm_rope_cache_write(q, k, v, q_weight, k_weight, eps, positions, inv_freq,
                             rot_dims: int, k_cache, v_cache, slot_mapping) -> torch.Tensor:
    """Per-head RMS norm of q [T, H, dim] and k [T, G, dim] (views into a merged
    projection are fine), rotation of the first ``rot_dims`` dims (dim i with
    i + rot_dims/2) in f32, one rounding; keys and v [T, Gv, vdim] stored in the
    paged cache.  Returns contiguous queries."""
    if q.numel() and _native_seq(q):
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
        _S.qk_norm_rope_cache_write(out, q, k, v, q_weight, k_weight, float(eps),
                                    positions, inv_freq, int(rot_dims), k_cache,
                                    v_cache, slot_mapping)
        return out
    return reference.qk_norm_rope_cache_write(q, k, v, q_weight, k_weight, eps, positions,
                                              inv_freq, rot_dims, k_cache, v_cache,
                                              slot_mapping)


def _chunk_matrix_core_fits(q, k_cache, v_cache, out, single: bool) -> bool:
    """The chunk variants of the MFMA kernels take bf16, equal key and value
    size of 128 (single queries: also 64), up to 8 query heads per key head, a
    whole number of key heads per value head, f32 output."""
    if _attn_ext() is None or _FORCE_REFERENCE or q.dtype != torch.bfloat16:
        return False
    d = q.shape[-1]
    kvh, vh = k_cache.shape[2], v_cache.shape[2]
    group = q.shape[1] // kvh
    return (d in ((64, 128) if single else (128,)) and v_cache.shape[-1] == d
            and 1 <= group <= 8 and q.shape[1] == group * kvh and kvh % vh == 0
            and q.is_contiguous() and out.is_contiguous())


def chunk_attention_uses_matrix_cores(dtype: torch.dtype, heads: int, kv_heads: int,
                                      dim: int, vdim: int) -> bool:
    """Shape test of the above without tensors (which extensions a model needs)."""
    return (dtype == torch.bfloat16 and dim == vdim and dim in (64, 128)
            and heads % kv_heads == 0 and 1 <= heads // kv_heads <= 8)


def chunk_attention_prefill(q, k_cache, v_cache, block_tables, query_start_loc,
                            seq_lens, scale, max_query_len, chunk: int,
                            out: torch.Tensor) -> torch.Tensor:
    """Causal grouped-query softmax attention of query portions over the paged
    cache where position i sees only the keys of its own chunk of ``chunk``
    positions (counted from position 0; 0 = no chunks).  The value cache may
    hold fewer heads than the key cache (key head g reads value head g mod
    Gv).  out [T, H, vdim] f32."""
    if q.numel() and _native_seq(q):
        if _chunk_matrix_core_fits(q, k_cache, v_cache, out, single=False):
            _attn_ext().chunk_attention_prefill(
                out, q, k_cache, v_cache, block_tables, query_start_loc, seq_lens,
                float(scale), int(max_query_len), int(chunk))
            return out
        _S.chunk_attention(out, q, k_cache, v_cache, block_tables, query_start_loc,
                           seq_lens, float(scale), int(max_query_len), int(chunk))
        return out
    out.copy_(reference.chunk_attention(q, k_cache, v_cache, block_tables.cpu(),
                                        query_start_loc.cpu(), seq_lens.cpu(), scale, chunk))
    return out


def chunk_attention_decode(q, k_cache, v_cache, block_tables, seq_lens, scale,
                           chunk: int, out: torch.Tensor) -> torch.Tensor:
    """Same attention for one new query per sequence (length 0 = padding row)."""
    if q.numel() and _native_seq(q):
        if _chunk_matrix_core_fits(q, k_cache, v_cache, out, single=True):
            _attn_ext().chunk_attention_decode(out, q, k_cache, v_cache, block_tables,
                                               seq_lens, float(scale), int(chunk))
            return out
        _S.chunk_attention(out, q, k_cache, v_cache, block_tables, None, seq_lens,
                           float(scale), 1, int(chunk))
        return out
    qsl = torch.arange(q.shape[0] + 1, dtype=torch.int32)
    out.copy_(reference.chunk_attention(q, k_cache, v_cache, block_tables.cpu(), qsl,
                                        seq_lens.cpu(), scale, chunk))
    return out


def diff_combine(a: torch.Tensor, lam: float, out_scale: float, eps: float,
                 gate: torch.Tensor | None, out_dtype: torch.dtype) -> torch.Tensor:
    """Differential attention's combination of two maps a [T, 2, H, vdim] f32:
    (a0 - lam * a1) / rms over vdim * out_scale * sigmoid(gate[t, h]) ->
    [T, H * vdim] in the compute dtype."""
    if a.numel() and _native_seq(a):
        t, _, h, dv = a.shape
        out = torch.empty((t, h * dv), dtype=out_dtype, device=a.device)
        _S.diff_combine(out, a, float(lam), float(out_scale), float(eps), gate)
        return out
    return reference.diff_combine(a, lam, out_scale, eps, gate, out_dtype)


def hgrn2_scan(q, f, v, f_bias, lower, state, seq_start_loc, seq_lens,
               state_slots) -> torch.Tensor:
    """HGRN2 recurrence over each sequence's new rows, f32 state [slots, H,
    vdim, dim] advanced in place; q, f [T, H, dim] and v [T, H, vdim] may be
    views into a merged projection.  Returns o [T, H * vdim] f32."""
    if q.numel() and _native_seq(q):
        o = torch.empty((q.shape[0], q.shape[1] * v.shape[-1]), dtype=torch.float32,
                        device=q.device)
        _S.hgrn2_scan(o, q, f, v, f_bias, lower, state, seq_start_loc, seq_lens,
                      state_slots)
        return o
    return reference.hgrn2_scan(q, f, v, f_bias, lower, state, seq_start_loc.cpu(),
                                seq_lens.cpu(), state_slots.cpu())


def group_rms_norm(y: torch.Tensor, weight: torch.Tensor, groups: int, eps: float,
                   out_dtype: torch.dtype) -> torch.Tensor:
    """RMS norm of f32 y [T, C] in ``groups`` equal parts, times weight [C]."""
    if y.numel() and _native_seq(y):
        out = torch.empty(y.shape, dtype=out_dtype, device=y.device)
        _S.group_rms_norm(out, y, weight, int(groups), float(eps))
        return out
    return reference.group_rms_norm(y, weight, groups, eps, out_dtype)


def moe_route_sigmoid(logits: torch.Tensor, top: int):
    """Sigmoid router: the ``top`` largest sigmoid(logits) per row, weighted by
    those scores as they are.  Returns (dense [T, E] f32, ids [T, top] int32,
    weights [T, top] f32)."""
    if logits.numel() and _native_seq(logits):
        t, n = logits.shape
        dev = logits.device
        dense = torch.empty((t, n), dtype=torch.float32, device=dev)
        ids = torch.empty((t, top), dtype=torch.int32, device=dev)
        w = torch.empty((t, top), dtype=torch.float32, device=dev)
        _S.moe_route_sigmoid(dense, ids, w, logits)
        return dense, ids, w
    return reference.moe_route_sigmoid(logits, top)


def silu_mul_scaled(gu: torch.Tensor, col_scale: torch.Tensor) -> torch.Tensor:
    """gu [T, E * 2 * ff] (per expert its gate rows, then its up rows) ->
    [T, E * ff]: silu(w * gate) * (w * up), w = col_scale[t, expert] f32."""
    if gu.numel() and _native_seq(gu):
        out = torch.empty((gu.shape[0], gu.shape[1] // 2), dtype=gu.dtype, device=gu.device)
        _S.silu_mul_scaled(out, gu, col_scale)
        return out
    return reference.silu_mul_scaled(gu, col_scale)
