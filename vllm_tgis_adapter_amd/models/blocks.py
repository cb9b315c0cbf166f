"""Building blocks for models that keep an f32 residual stream.

Each block is one mechanism with its constants as constructor parameters, so
that another design can assemble them differently:

- ``StreamRMSNorm``     RMS norm of the f32 stream, weight applied as (offset + w)
- ``ShortConv``         depthwise causal convolution over time whose last
                        taps-1 inputs are per-sequence state
- ``LatentAttention``   multi-head attention whose keys and values are
                        up-projections of one cached latent row per token, with
                        a rotated key part shared by all heads, an optional
                        sliding window and a per-head sink in the softmax
- ``DenseMLP``          down(act(up(h))) with the tanh-form GELU
- ``TokenSideInput``    gated per-layer token embedding added to the stream
                        through its own RMS norm
- ``StreamLayerNorm``   bias-free layer norm of the f32 stream
- ``GatedDenseMLP``     down(act(gate(h)) * up(h)) with the tanh-form GELU
- ``QKNormAttention``   grouped-query softmax attention over the paged cache,
                        per-head RMS norm on queries and keys, no rotation, an
                        optional position-dependent query temperature; the
                        value size may differ from the query/key size
- ``SSDMixer``          state-space-duality recurrence (short convolution,
                        per-head scalar decay, gated grouped RMS norm)
- ``RGLRUMixer``        recurrent block with a real-gated linear recurrent unit
- ``MLSTMMixer``        matrix memory with exponential gating
- ``ParallelMixer``     two mixers fed one input through a single merged
                        projection, their outputs mixed with fixed scales
- ``scaled_rotary_frequencies``  rotation frequencies with the ramped
                        (YaRN-style) stretch of the slowly turning pairs
- ``RotatedAttention``  grouped-query softmax attention with rotated queries
                        and keys (half-split or interleaved pairs), an optional
                        sliding window, an optional sink in the softmax
                        denominator, values that may be the unrotated keys, and
                        an optional sigmoid output gate
- ``BiasedDenseMLP``    down(act(up h + b) ) + b with a squared relu
- ``RoutedExperts``     softmax router with a choice correction, top-k of
                        small squared-relu experts plus identity experts
- ``TokenShift``        per-channel blend of a row of the f32 stream with the
                        row before it, the last row carried per sequence
- ``DiffAttention``     differential grouped-query attention: two softmax maps
                        over the same values, query/key norm, rotation with
                        piecewise frequency scaling, a chunk mask, a per-head
                        sigmoid gate
- ``HGRN2Mixer``        gated linear recurrence whose forget gate (with a
                        per-channel lower bound) also sets what is written
- ``GatedRoutedExperts`` sigmoid router, top-k of small gated (silu) experts
                        whose input is multiplied by the routing weight
- ``stepped_rotary_frequencies``  rotation frequencies divided by a factor
                        for long wavelengths, kept for short ones, blended
                        linearly in between

The recurrent mixers keep their state (f32) and the last inputs of their short
convolutions in per-sequence slots; a sequence that starts in a step starts
from zero state whatever its slot held before.

The stream itself, norms, rotation angles, attention scores and softmax are
f32 whatever the compute dtype is; projections run in the compute dtype.
"""

from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from .. import ops
from ..engine.metadata import AttnMetadata
from ..parallel import divide, get_tp_rank, get_tp_world_size
from ..parallel.layers import ColumnParallelLinear, RowParallelLinear


def _f32_param(*shape, fill: float = 0.0) -> nn.Parameter:
    return nn.Parameter(torch.full(shape, fill, dtype=torch.float32), requires_grad=False)


class StreamRMSNorm(nn.Module):
    """f32 stream -> compute dtype: x / sqrt(mean(x^2) + eps) * (offset + w)."""

    def __init__(self, width: int, eps: float, weight_offset: float, dtype: torch.dtype):
        super().__init__()
        self.eps = eps
        self.weight_offset = weight_offset
        self.dtype = dtype
        self.weight = _f32_param(width, fill=1.0 - weight_offset)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.rms_norm_stream(x, self.weight, self.eps, self.weight_offset, self.dtype)


class ShortConv(nn.Module):
    """h + conv(h): per-channel causal convolution over time, ``taps`` taps,
    no bias.  The last taps-1 inputs of a sequence are carried in a state
    slot so that a sequence can be fed in portions of any size."""

    def __init__(self, width: int, taps: int):
        super().__init__()
        self.width = width
        self.taps = taps
        w = torch.empty(width, taps, dtype=torch.float32).normal_(0.0, 0.1)
        self.weight = nn.Parameter(w, requires_grad=False)

    def state_shape(self) -> tuple:
        return (max(self.taps - 1, 0), self.width)

    def forward(self, h: torch.Tensor, state: torch.Tensor, meta: AttnMetadata) -> torch.Tensor:
        return ops.causal_conv_state(
            h, self.weight, state, meta.seq_start_loc, meta.seq_lens,
            meta.state_slots, add_input=True)


def scaled_rotary_frequencies(base: float, dims: int,
                              scaling: Optional[dict] = None) -> tuple[list, float]:
    """Frequencies of the dims/2 rotated pairs, f_i = base^(-2i/dims), and the
    factor that multiplies cos and sin (1 without scaling).

    ``scaling`` = {factor s, original L, fast, slow} stretches the context by s
    the YaRN way: pair i makes L f_i / 2 pi turns over the original length; the
    pair index at which that count equals t is p(t) = dims ln(L / (2 pi t)) /
    (2 ln base).  With lo = max(floor(p(fast)), 0), hi = min(ceil(p(slow)),
    dims - 1) and ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1) the
    frequency becomes f_i / s * ramp_i + f_i * (1 - ramp_i): fast pairs keep
    their frequency, slow pairs are interpolated.  cos and sin are multiplied
    by 0.1 ln(s) + 1.  All of it in float64; callers round once to f32."""
    import math

    half = dims // 2
    freqs = [float(base) ** (-2.0 * i / dims) for i in range(half)]
    if not scaling:
        return freqs, 1.0
    s = float(scaling["factor"])
    orig = float(scaling["original"])

    def pair_at(turns: float) -> float:
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(float(base)))

    lo = max(math.floor(pair_at(float(scaling["fast"]))), 0)
    hi = min(math.ceil(pair_at(float(scaling["slow"]))), dims - 1)
    out = []
    for i, f in enumerate(freqs):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / s * ramp + f * (1.0 - ramp))
    return out, 0.1 * math.log(s) + 1.0


class LatentAttention(nn.Module):
    """Attention over a cached latent.

    Per token the cache holds one row [rank + rot]: the RMS-normed latent c
    and a rotated key part shared by all heads.  Head h's key is
    [W_uk[h] c ; k_rot] and its value W_uv[h] c.  The kernels work in latent
    space: the unrotated query is folded through W_uk[h] first
    (q_lat = W_uk[h]^T q), scores are (q_lat . c + q_rot . k_rot) * scale, the
    weighted sum of c is unfolded through W_uv[h] afterwards — every head
    reads the same single row per token.

    ``kv_owner`` False: the layer has no down-projection of its own and reads
    the rows another layer wrote this step (its cache tensor is that layer's).
    """

    def __init__(self, width: int, *, heads: int, dim: int, rot_dim: int, vdim: int,
                 rank: int, scale: float, window: int, rot_base: float,
                 rot_dims: int, eps: float, kv_owner: bool, has_sink: bool,
                 dtype: torch.dtype, rot_interleaved: bool = False,
                 rot_scaling: Optional[dict] = None, head_gate: bool = False,
                 two_term_weights: bool = False, q_rank: int = 0):
        """``q_rank`` > 0: queries go through a latent of that size, q = W_uq
        rmsnorm(W_dq h) (plain weight, eps of the layer).
        ``rot_interleaved``: dim 2i is paired with 2i+1 instead of i with
        i + rot_dims/2.  ``rot_scaling``: see ``scaled_rotary_frequencies``.
        ``head_gate``: head h's output is multiplied by sigmoid(W_g x)_h.
        ``two_term_weights``: the bf16 matrix-core kernel feeds the softmax
        weights to the value product as two bf16 terms (16 mantissa bits)."""
        super().__init__()
        tp = get_tp_world_size()
        self.heads = divide(heads, tp)
        self.dim, self.rot_dim, self.vdim, self.rank = dim, rot_dim, vdim, rank
        self.scale, self.window, self.eps = scale, window, eps
        self.rot_dims = rot_dims
        self.kv_owner = kv_owner
        self.dtype = dtype
        self.q_rank = q_rank
        self.q_proj = ColumnParallelLinear(q_rank or width, heads * (dim + rot_dim), dtype=dtype)
        if q_rank:
            # replicated on every rank, like the key/value latent
            self.dq_weight = nn.Parameter(
                torch.empty(q_rank, width, dtype=dtype).normal_(0.0, 0.02), requires_grad=False)
            self.dq_norm = _f32_param(q_rank, fill=1.0)
        self.o_proj = RowParallelLinear(heads * vdim, width, dtype=dtype)
        if kv_owner:
            # replicated on every rank: the latent is shared by all heads.  With a
            # head gate this rank's gate rows follow the down-projection's, so
            # that one product yields both
            self.dkv_weight = nn.Parameter(
                torch.empty(rank + rot_dim + (self.heads if head_gate else 0), width,
                            dtype=dtype).normal_(0.0, 0.02),
                requires_grad=False)
            self.dkv_norm = _f32_param(rank, fill=1.0)
        # [H, dim, rank] and [H, rank, vdim] for the batched fold / unfold
        self.uk = nn.Parameter(
            torch.empty(self.heads, dim, rank, dtype=dtype).normal_(0.0, 0.02),
            requires_grad=False)
        self.uv_t = nn.Parameter(
            torch.empty(self.heads, rank, vdim, dtype=dtype).normal_(0.0, 0.02),
            requires_grad=False)
        self.sink = _f32_param(self.heads) if has_sink else None
        self.rot_interleaved = rot_interleaved
        self.two_term_weights = two_term_weights
        freqs, self.rot_mag = scaled_rotary_frequencies(rot_base, rot_dims, rot_scaling)
        self.register_buffer(
            "inv_freq", torch.tensor(freqs, dtype=torch.float64).to(torch.float32),
            persistent=False)
        self.head_gate = head_gate
        # a layer without a down-projection of its own keeps its gate rows apart
        self.gate_weight = (
            nn.Parameter(torch.empty(self.heads, width, dtype=dtype).normal_(0.0, 0.02),
                         requires_grad=False) if head_gate and not kv_owner else None)

    # -- weights -----------------------------------------------------------
    def load(self, q, dkv, dkv_norm, uk, uv, sink, o, gate=None, dq=None,
             dq_norm=None) -> None:
        r, h = get_tp_rank(), self.heads
        self.q_proj.load_full_weight(q)
        if self.q_rank:
            self.dq_weight.data.copy_(dq.to(self.dtype))
            self.dq_norm.data.copy_(dq_norm.float())
        self.o_proj.load_full_weight(o)
        if self.gate_weight is not None:
            self.gate_weight.data.copy_(gate[r * h:(r + 1) * h].to(self.dtype))
        if self.kv_owner:
            n = self.rank + self.rot_dim
            self.dkv_weight.data[:n].copy_(dkv.to(self.dtype))
            if self.head_gate:
                self.dkv_weight.data[n:].copy_(gate[r * h:(r + 1) * h].to(self.dtype))
            self.dkv_norm.data.copy_(dkv_norm.float())
        uk = uk.view(-1, self.dim, self.rank)[r * h:(r + 1) * h]
        uv = uv.view(-1, self.vdim, self.rank)[r * h:(r + 1) * h]
        self.uk.data.copy_(uk.to(self.dtype))
        self.uv_t.data.copy_(uv.transpose(1, 2).to(self.dtype))
        if self.sink is not None:
            self.sink.data.copy_(sink.float()[r * h:(r + 1) * h])

    # -- forward -----------------------------------------------------------
    def forward(self, h: torch.Tensor, positions: torch.Tensor,
                cache: torch.Tensor, meta: AttnMetadata) -> torch.Tensor:
        t = h.shape[0]
        nh, d, r, rank = self.heads, self.dim, self.rot_dim, self.rank
        if self.q_rank:
            cq = ops.group_rms_norm(ops.linear(h, self.dq_weight), self.dq_norm, 1,
                                    self.eps, self.dtype)
            q = self.q_proj(cq).view(t, nh, d + r)
        else:
            q = self.q_proj(h).view(t, nh, d + r)
        if self.rot_dims:
            ops.rope_partial(q, positions, self.inv_freq, d, self.rot_dims,
                             self.rot_interleaved, self.rot_mag)
        g = None
        if self.kv_owner:
            dkv = ops.linear(h, self.dkv_weight)
            if self.head_gate:
                dkv, g = dkv[:, :rank + r], dkv[:, rank + r:]
            ops.latent_kv_write(dkv, self.dkv_norm, self.eps, positions,
                                self.inv_freq, self.rot_dims, cache,
                                meta.slot_mapping, self.rot_interleaved, self.rot_mag)
        # fold the unrotated query into latent space: [H, T, rank]
        q_lat = torch.bmm(q[:, :, :d].transpose(0, 1), self.uk).transpose(0, 1)
        q_rot = q[:, :, d:]
        o_lat = torch.empty((nh, t, rank), dtype=h.dtype, device=h.device)
        o_view = o_lat.transpose(0, 1)   # [T, H, rank]
        npt = meta.num_prefill_tokens
        if npt:
            ops.latent_attention_prefill(
                q_lat[:npt], q_rot[:npt], cache, meta.prefill_block_tables,
                meta.prefill_query_start_loc, meta.prefill_seq_lens, self.scale,
                self.window, self.sink, meta.max_prefill_query_len,
                out=o_view[:npt], two_term=self.two_term_weights)
        if meta.num_decode_seqs:
            ops.latent_attention_decode(
                q_lat[npt:], q_rot[npt:], cache, meta.decode_block_tables,
                meta.decode_seq_lens, self.scale, self.window, self.sink,
                out=o_view[npt:], two_term=self.two_term_weights)
        o = torch.bmm(o_lat, self.uv_t)                    # [H, T, vdim]
        if self.head_gate:
            # gate and the [H, T] -> [T, H] regrouping in one pass
            if g is None:
                g = ops.linear(h, self.gate_weight)        # [T, H]
            return self.o_proj(ops.sigmoid_gate_mul(o.transpose(0, 1), g))
        return self.o_proj(o.transpose(0, 1).reshape(t, nh * self.vdim))


class DenseMLP(nn.Module):
    def __init__(self, width: int, ff: int, dtype: torch.dtype):
        super().__init__()
        self.up = ColumnParallelLinear(width, ff, dtype=dtype)
        self.down = RowParallelLinear(ff, width, dtype=dtype)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return self.down(ops.gelu_tanh(self.up(h)))


class TokenSideInput(nn.Module):
    """x <- x + mult * rmsnorm(proj(gelu_tanh(gate x) * e)) * w, e being this
    layer's slice of a per-token side embedding."""

    def __init__(self, width: int, side_dim: int, eps: float, mult: float,
                 dtype: torch.dtype):
        super().__init__()
        self.eps, self.mult = eps, mult
        self.gate = nn.Parameter(
            torch.empty(side_dim, width, dtype=dtype).normal_(0.0, 0.02), requires_grad=False)
        self.proj = nn.Parameter(
            torch.empty(width, side_dim, dtype=dtype).normal_(0.0, 0.02), requires_grad=False)
        self.norm = _f32_param(width, fill=1.0)

    def forward(self, x: torch.Tensor, x_cast: torch.Tensor, e: torch.Tensor,
                next_norm: "StreamRMSNorm | None" = None):
        """Updates x in place; with ``next_norm`` the norm that reads the
        updated stream next is computed in the same kernel and returned."""
        g = ops.gelu_tanh(ops.linear(x_cast, self.gate), mul=e)
        y = ops.linear(g, self.proj)
        nn_ = None
        if next_norm is not None:
            nn_ = (next_norm.weight, next_norm.eps, next_norm.weight_offset, next_norm.dtype)
        return ops.stream_add_rms_norm(x, y, self.norm, self.eps, self.mult, nn_)


# ---------------------------------------------------------------------------
# Layer-norm stream blocks, softmax attention with query/key norm, recurrent
# mixers.  Mixers share one shape: ``in_rows`` rows of an input projection
# (own weight, or a slice of a merged one when ``own_in`` is False), ``mix``
# from the projected rows to the rows that ``o_weight`` maps back to the
# width, and ``cache_shapes`` naming what they keep per cache block / slot.
# ---------------------------------------------------------------------------


def _randn_param(shape, dtype, std: float = 0.02) -> nn.Parameter:
    return nn.Parameter(torch.empty(*shape, dtype=dtype).normal_(0.0, std),
                        requires_grad=False)


class StreamLayerNorm(nn.Module):
    """f32 stream -> compute dtype: (x - mean) / sqrt(var + eps) * w, no bias."""

    def __init__(self, width: int, eps: float, dtype: torch.dtype):
        super().__init__()
        self.eps = eps
        self.dtype = dtype
        self.weight = _f32_param(width, fill=1.0)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.layer_norm_stream(x, self.weight, self.eps, self.dtype)

    def as_next(self):
        return (self.weight, self.eps, self.dtype)


class GatedDenseMLP(nn.Module):
    """down(gelu_tanh(gate h) * (up h)); gate and up are one merged product."""

    def __init__(self, width: int, ff: int, dtype: torch.dtype):
        super().__init__()
        if get_tp_world_size() != 1:
            raise ValueError("GatedDenseMLP is not sharded; run it with one rank")
        self.ff = ff
        self.gate_up = _randn_param((2 * ff, width), dtype)
        self.down = _randn_param((width, ff), dtype)

    def load(self, gate, up, down) -> None:
        self.gate_up.data[:self.ff].copy_(gate.to(self.gate_up.dtype))
        self.gate_up.data[self.ff:].copy_(up.to(self.gate_up.dtype))
        self.down.data.copy_(down.to(self.down.dtype))

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        gu = ops.linear(h, self.gate_up)
        a = ops.gelu_tanh(gu[:, :self.ff], mul=gu[:, self.ff:])
        return ops.linear(a, self.down)


class _Mixer(nn.Module):
    """Common shape of the mixers below (see the section comment)."""

    in_rows: int
    out_rows: int
    has_in_bias = False

    def _alloc(self, width: int, own_in: bool, dtype: torch.dtype) -> None:
        if get_tp_world_size() != 1:
            raise ValueError(f"{type(self).__name__} is not sharded; run it with one rank")
        self.width = width
        self.dtype = dtype
        self.in_weight = _randn_param((self.in_rows, width), dtype) if own_in else None
        self.in_bias = (nn.Parameter(torch.zeros(self.in_rows, dtype=dtype), requires_grad=False)
                        if own_in and self.has_in_bias else None)
        self.o_weight = _randn_param((width, self.out_rows), dtype)

    def project(self, h: torch.Tensor) -> torch.Tensor:
        return ops.linear(h, self.in_weight, self.in_bias)

    def forward(self, h, positions, cache, meta: AttnMetadata) -> torch.Tensor:
        return ops.linear(self.mix(self.project(h), positions, cache, meta), self.o_weight)

    def load_in(self, weight: torch.Tensor, bias, tensors: dict) -> None:
        raise NotImplementedError

    def load(self, tensors: dict) -> None:
        """tensors: this mixer's checkpoint tensors by their short names."""
        self.load_in(self.in_weight.data, None if self.in_bias is None else self.in_bias.data,
                     tensors)
        self.o_weight.data.copy_(tensors["o"].to(self.dtype))
        self.load_rest(tensors)

    def load_rest(self, tensors: dict) -> None:
        pass

    # what the mixer keeps: {name: (kind, shape-per-block-or-slot, dtype)} with
    # kind "paged" (per cache block) or "slot" (per sequence)
    def cache_shapes(self, block_size: int) -> list:
        return []


class QKNormAttention(_Mixer):
    """Causal grouped-query softmax attention.  q, k are RMS-normed per head
    with a weight shared by all heads (plain weight); positions enter only
    through the optional query temperature 1 + coef * ln(floor((p + 1) /
    every) + 1); score = q . k * scale.  Projected rows: [q | k | v]."""

    def __init__(self, width: int, *, heads: int, kv_heads: int, dim: int, vdim: int,
                 scale: float, eps: float, temp_coef: float = 0.0, temp_every: int = 0,
                 own_in: bool = True, dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        if heads % kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        self.heads, self.kv_heads, self.dim, self.vdim = heads, kv_heads, dim, vdim
        self.scale, self.eps = scale, eps
        self.temp_coef, self.temp_every = temp_coef, temp_every
        self.in_rows = heads * dim + kv_heads * (dim + vdim)
        self.out_rows = heads * vdim
        self._alloc(width, own_in, dtype)
        self.q_norm = _f32_param(dim, fill=1.0)
        self.k_norm = _f32_param(dim, fill=1.0)

    def load_in(self, weight, bias, t) -> None:
        a = self.heads * self.dim
        b = a + self.kv_heads * self.dim
        weight[:a].copy_(t["q"].to(weight.dtype))
        weight[a:b].copy_(t["k"].to(weight.dtype))
        weight[b:].copy_(t["v"].to(weight.dtype))

    def load_rest(self, t) -> None:
        self.q_norm.data.copy_(t["q.norm"].float())
        self.k_norm.data.copy_(t["k.norm"].float())

    def cache_shapes(self, block_size: int) -> list:
        return [("paged", (block_size, self.kv_heads, self.dim), self.dtype),
                ("paged", (block_size, self.kv_heads, self.vdim), self.dtype)]

    def mix(self, proj, positions, cache, meta: AttnMetadata) -> torch.Tensor:
        t = proj.shape[0]
        nh, ng, d, dv = self.heads, self.kv_heads, self.dim, self.vdim
        a = nh * d
        b = a + ng * d
        k_cache, v_cache = cache
        q = ops.qk_norm_cache_write(
            proj[:, :a].view(t, nh, d), proj[:, a:b].view(t, ng, d),
            proj[:, b:].view(t, ng, dv), self.q_norm, self.k_norm, self.eps,
            positions, self.temp_coef, self.temp_every, k_cache, v_cache,
            meta.slot_mapping)
        out = torch.empty((t, nh, dv), dtype=proj.dtype, device=proj.device)
        npt = meta.num_prefill_tokens
        if npt:
            ops.gqa_attention_prefill(
                q[:npt], k_cache, v_cache, meta.prefill_block_tables,
                meta.prefill_query_start_loc, meta.prefill_seq_lens, self.scale,
                meta.max_prefill_query_len, out=out[:npt])
        if meta.num_decode_seqs:
            ops.gqa_attention_decode(
                q[npt:], k_cache, v_cache, meta.decode_block_tables,
                meta.decode_seq_lens, self.scale, out=out[npt:])
        return out.view(t, nh * dv)


class SSDMixer(_Mixer):
    """State-space-duality mixer.  Projected rows: [z | x | B | C | dt] with
    inner = heads * vdim, B and C of groups * state each.  x, B, C pass a short
    causal convolution with bias and silu; dt = softplus(dt + dt_bias); per
    head S_t = exp(-exp(A_log) dt) S_(t-1) + dt B_t x_t^T, y_t = S_t^T C_t + D
    x_t; y * silu(z) is RMS-normed in ``norm_groups`` parts, times a weight."""

    def __init__(self, width: int, *, heads: int, vdim: int, state: int, groups: int,
                 taps: int, norm_groups: int, eps: float, own_in: bool = True,
                 dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        if heads % groups or (heads * vdim) % norm_groups:
            raise ValueError("heads must divide by groups, inner size by norm_groups")
        self.heads, self.vdim, self.nstate, self.groups = heads, vdim, state, groups
        self.taps, self.norm_groups, self.eps = taps, norm_groups, eps
        self.inner = heads * vdim
        self.conv_ch = self.inner + 2 * groups * state
        self.in_rows = self.inner + self.conv_ch + heads
        self.out_rows = self.inner
        self._alloc(width, own_in, dtype)
        self.conv_weight = nn.Parameter(
            torch.empty(self.conv_ch, taps, dtype=torch.float32).normal_(0.0, 0.2),
            requires_grad=False)
        self.conv_bias = _f32_param(self.conv_ch)
        # step sizes around 0.01..0.1 and decays A in 1..16 for random weights
        self.dt_bias = nn.Parameter(torch.empty(heads).uniform_(-4.6, -2.2), requires_grad=False)
        self.a_log = nn.Parameter(torch.empty(heads).uniform_(0.0, 2.77), requires_grad=False)
        self.d_skip = _f32_param(heads, fill=1.0)
        self.norm = _f32_param(self.inner, fill=1.0)

    def load_in(self, weight, bias, t) -> None:
        weight.copy_(t["in"].to(weight.dtype))

    def load_rest(self, t) -> None:
        self.conv_weight.data.copy_(t["conv"].float())
        self.conv_bias.data.copy_(t["conv.b"].float())
        self.dt_bias.data.copy_(t["dt_bias"].float())
        self.a_log.data.copy_(t["A_log"].float())
        self.d_skip.data.copy_(t["D"].float())
        self.norm.data.copy_(t["norm"].float())

    def cache_shapes(self, block_size: int) -> list:
        return [("slot", (max(self.taps - 1, 0), self.conv_ch), self.dtype),
                ("slot", (self.heads, self.vdim, self.nstate), torch.float32)]

    def mix(self, proj, positions, cache, meta: AttnMetadata) -> torch.Tensor:
        conv_state, ssm_state = cache
        inner = self.inner
        z = proj[:, :inner]
        xbc = ops.causal_conv_state(
            proj[:, inner:inner + self.conv_ch], self.conv_weight, conv_state,
            meta.seq_start_loc, meta.seq_lens, meta.state_slots, add_input=False,
            bias=self.conv_bias, act="silu")
        y = ops.ssd_scan(xbc, proj[:, inner + self.conv_ch:], self.dt_bias, self.a_log,
                         self.d_skip, ssm_state, meta.seq_start_loc, meta.seq_lens,
                         meta.state_slots, self.heads, self.vdim, self.nstate, self.groups)
        return ops.gated_group_norm(y, z, self.norm, self.norm_groups, self.eps,
                                    gate_first=True, out_dtype=self.dtype)


class RGLRUMixer(_Mixer):
    """Recurrent block: y = gelu_tanh(W_y h + b), u = conv(W_x h + b) (short
    causal convolution with bias, no activation); per block of channels r =
    sigmoid(R_a u + b), i = sigmoid(R_i u + b); a = exp(-c r softplus(lam)),
    S_t = a S_(t-1) + sqrt(1 - a^2) i u; output rows S * y.  Projected rows:
    [y | x]."""

    has_in_bias = True

    def __init__(self, width: int, *, rec_width: int, blocks: int, taps: int,
                 gate_c: float = 8.0, own_in: bool = True,
                 dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        if rec_width % blocks:
            raise ValueError("recurrent width must divide by blocks")
        self.rec_width, self.blocks, self.taps, self.gate_c = rec_width, blocks, taps, gate_c
        self.in_rows = 2 * rec_width
        self.out_rows = rec_width
        self._alloc(width, own_in, dtype)
        bw = rec_width // blocks
        self.conv_weight = nn.Parameter(
            torch.empty(rec_width, taps, dtype=torch.float32).normal_(0.0, 0.2),
            requires_grad=False)
        self.conv_bias = _f32_param(rec_width)
        # stored transposed ([block, in, out]) for the batched product
        self.ra_t = _randn_param((blocks, bw, bw), dtype, std=bw ** -0.5)
        self.ri_t = _randn_param((blocks, bw, bw), dtype, std=bw ** -0.5)
        self.ra_bias = _f32_param(rec_width)
        self.ri_bias = _f32_param(rec_width)
        self.lam = nn.Parameter(torch.empty(rec_width).uniform_(-4.0, -1.0), requires_grad=False)

    def load_in(self, weight, bias, t) -> None:
        w = self.rec_width
        weight[:w].copy_(t["y"].to(weight.dtype))
        weight[w:].copy_(t["x"].to(weight.dtype))
        bias[:w].copy_(t["y.b"].to(bias.dtype))
        bias[w:].copy_(t["x.b"].to(bias.dtype))

    def load_rest(self, t) -> None:
        self.conv_weight.data.copy_(t["conv"].float())
        self.conv_bias.data.copy_(t["conv.b"].float())
        self.ra_t.data.copy_(t["ra"].transpose(1, 2).to(self.dtype))
        self.ri_t.data.copy_(t["ri"].transpose(1, 2).to(self.dtype))
        self.ra_bias.data.copy_(t["ra.b"].float().reshape(-1))
        self.ri_bias.data.copy_(t["ri.b"].float().reshape(-1))
        self.lam.data.copy_(t["lam"].float())

    def cache_shapes(self, block_size: int) -> list:
        return [("slot", (max(self.taps - 1, 0), self.rec_width), self.dtype),
                ("slot", (self.rec_width,), torch.float32)]

    def mix(self, proj, positions, cache, meta: AttnMetadata) -> torch.Tensor:
        conv_state, rec_state = cache
        t, w, nb = proj.shape[0], self.rec_width, self.blocks
        yb = ops.gelu_tanh(proj[:, :w])
        u = ops.causal_conv_state(
            proj[:, w:], self.conv_weight, conv_state, meta.seq_start_loc,
            meta.seq_lens, meta.state_slots, add_input=False, bias=self.conv_bias)
        ub = u.view(t, nb, w // nb).transpose(0, 1)              # [blocks, T, bw]
        r_pre = torch.bmm(ub, self.ra_t).transpose(0, 1).reshape(t, w)
        i_pre = torch.bmm(ub, self.ri_t).transpose(0, 1).reshape(t, w)
        return ops.rglru_scan(u, r_pre, i_pre, self.ra_bias, self.ri_bias, self.lam,
                              self.gate_c, yb, rec_state, meta.seq_start_loc,
                              meta.seq_lens, meta.state_slots)


class MLSTMMixer(_Mixer):
    """Matrix memory with exponential gating.  q = W_q h / sqrt(dim), k, v per
    head; log input gate i = cap tanh((W_i h + b) / cap), log forget gate f =
    logsigmoid(cap tanh((W_f h + b) / cap)); running maximum m, initialised
    to 0: m_t = max(f + m, i), S_t = exp(f + m - m_t) S + exp(i - m_t) k v^T, n
    likewise with k; o = S^T q / (max(|n . q|, exp(-m_t)) + 1e-6); each head's o
    is RMS-normed, times a weight, times sigmoid(W_g h).  Projected rows:
    [q | k | v | g | i | f]."""

    def __init__(self, width: int, *, heads: int, dim: int, vdim: int, gate_cap: float,
                 eps: float, own_in: bool = True, dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        self.heads, self.dim, self.vdim = heads, dim, vdim
        self.gate_cap, self.eps = gate_cap, eps
        self.in_rows = 2 * heads * dim + 2 * heads * vdim + 2 * heads
        self.out_rows = heads * vdim
        self._alloc(width, own_in, dtype)
        self.i_bias = _f32_param(heads)
        self.f_bias = _f32_param(heads, fill=3.0)
        self.norm = _f32_param(heads * vdim, fill=1.0)

    def load_in(self, weight, bias, t) -> None:
        off = 0
        for name in ("q", "k", "v", "g", "i", "f"):
            n = t[name].shape[0]
            weight[off:off + n].copy_(t[name].to(weight.dtype))
            off += n

    def load_rest(self, t) -> None:
        self.i_bias.data.copy_(t["i.b"].float())
        self.f_bias.data.copy_(t["f.b"].float())
        self.norm.data.copy_(t["norm"].float())

    def cache_shapes(self, block_size: int) -> list:
        return [("slot", (self.heads, self.vdim, self.dim), torch.float32),
                ("slot", (self.heads, self.dim), torch.float32),
                ("slot", (self.heads,), torch.float32)]

    def mix(self, proj, positions, cache, meta: AttnMetadata) -> torch.Tensor:
        s_state, n_state, m_state = cache
        t, nh, d, dv = proj.shape[0], self.heads, self.dim, self.vdim
        a = nh * d
        b = 2 * a
        c = b + nh * dv
        e = c + nh * dv
        o = ops.mlstm_scan(
            proj[:, :a].view(t, nh, d), proj[:, a:b].view(t, nh, d),
            proj[:, b:c].view(t, nh, dv), proj[:, e:e + nh], proj[:, e + nh:],
            self.i_bias, self.f_bias, self.gate_cap, d ** -0.5, s_state, n_state,
            m_state, meta.seq_start_loc, meta.seq_lens, meta.state_slots)
        return ops.gated_group_norm(o, proj[:, c:e], self.norm, nh, self.eps,
                                    gate_first=False, out_dtype=self.dtype)


class ParallelMixer(nn.Module):
    """Two mixers fed one input through a single merged projection; result =
    left_scale * left + right_scale * right.  Returns the two outputs
    and their scales; the caller's residual kernel forms the sum in f32."""

    def __init__(self, width: int, left: _Mixer, right: _Mixer, left_scale: float,
                 right_scale: float, dtype: torch.dtype):
        super().__init__()
        if left.has_in_bias or right.has_in_bias:
            raise ValueError("merged projection of mixers with input bias is not supported")
        self.left, self.right = left, right
        self.left_scale, self.right_scale = left_scale, right_scale
        self.in_weight = _randn_param((left.in_rows + right.in_rows, width), dtype)

    def load(self, left_tensors: dict, right_tensors: dict) -> None:
        n = self.left.in_rows
        for mod, rows, t in ((self.left, self.in_weight.data[:n], left_tensors),
                             (self.right, self.in_weight.data[n:], right_tensors)):
            mod.load_in(rows, None, t)
            mod.o_weight.data.copy_(t["o"].to(mod.dtype))
            mod.load_rest(t)

    def cache_shapes(self, block_size: int) -> list:
        return self.left.cache_shapes(block_size) + self.right.cache_shapes(block_size)

    def forward(self, h, positions, cache, meta: AttnMetadata):
        proj = ops.linear(h, self.in_weight)
        n = self.left.in_rows
        nl = len(self.left.cache_shapes(1))
        a = ops.linear(self.left.mix(proj[:, :n], positions, cache[:nl], meta),
                       self.left.o_weight)
        b = ops.linear(self.right.mix(proj[:, n:], positions, cache[nl:], meta),
                       self.right.o_weight)
        return a, b


class RotatedAttention(_Mixer):
    """Causal grouped-query softmax attention with rotary positions.

    Projected rows: [q | k | v? | gate?].  The first ``rot_dims`` dims of every
    query and key head are rotated (pairs (i, i + rot_dims/2), or (2i, 2i+1)
    when ``rot_interleaved``); score = q . k * scale; a query at position i
    sees keys j with 0 <= i - j < window (window 0: every j <= i); with
    ``sink`` (a logit) the softmax denominator also holds exp(sink), a key
    that has no value.  ``values_from_keys``: there is no value projection,
    the values are the keys as projected, before rotation (vdim = dim).
    ``gate`` "elementwise": the concatenated heads are multiplied by
    sigmoid(W_g h) before the output projection."""

    def __init__(self, width: int, *, heads: int, kv_heads: int, dim: int, vdim: int,
                 scale: float, window: int = 0, sink: Optional[float] = None,
                 rot_base: float = 10000.0, rot_dims: int = 0,
                 rot_interleaved: bool = False, rot_scaling: Optional[dict] = None,
                 values_from_keys: bool = False, gate: Optional[str] = None,
                 own_in: bool = True, dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        if heads % kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        if values_from_keys and vdim != dim:
            raise ValueError("values taken from the keys have the key size")
        if gate not in (None, "elementwise"):
            raise ValueError(f"unknown gate {gate!r}")
        if rot_dims % 2 or rot_dims > dim:
            raise ValueError("rot_dims must be even and at most dim")
        self.heads, self.kv_heads, self.dim, self.vdim = heads, kv_heads, dim, vdim
        self.scale, self.window, self.sink = scale, window, sink
        self.rot_dims, self.rot_interleaved = rot_dims, rot_interleaved
        self.values_from_keys, self.gate = values_from_keys, gate
        self.in_rows = (heads * dim + kv_heads * dim
                        + (0 if values_from_keys else kv_heads * vdim)
                        + (heads * vdim if gate else 0))
        self.out_rows = heads * vdim
        self._alloc(width, own_in, dtype)
        freqs, self.rot_mag = scaled_rotary_frequencies(rot_base, max(rot_dims, 2), rot_scaling)
        self.register_buffer(
            "inv_freq", torch.tensor(freqs, dtype=torch.float64).to(torch.float32),
            persistent=False)

    def load_in(self, weight, bias, t) -> None:
        off = 0
        names = ["q", "k"] + ([] if self.values_from_keys else ["v"]) + (["g"] if self.gate else [])
        for name in names:
            n = t[name].shape[0]
            weight[off:off + n].copy_(t[name].to(weight.dtype))
            off += n
        if off != self.in_rows:
            raise ValueError("projection tensors do not add up to the mixer's rows")

    def cache_shapes(self, block_size: int) -> list:
        return [("paged", (block_size, self.kv_heads, self.dim), self.dtype),
                ("paged", (block_size, self.kv_heads, self.vdim), self.dtype)]

    def mix(self, proj, positions, cache, meta: AttnMetadata) -> torch.Tensor:
        t = proj.shape[0]
        nh, ng, d, dv = self.heads, self.kv_heads, self.dim, self.vdim
        a = nh * d
        b = a + ng * d
        k_cache, v_cache = cache
        k = proj[:, a:b].view(t, ng, d)
        if self.values_from_keys:
            v, c = k, b
        else:
            c = b + ng * dv
            v = proj[:, b:c].view(t, ng, dv)
        q = ops.rope_kv_cache_write(
            proj[:, :a].view(t, nh, d), k, v, positions, self.inv_freq, self.rot_dims,
            self.rot_interleaved, self.rot_mag, k_cache, v_cache, meta.slot_mapping)
        out = torch.empty((t, nh, dv), dtype=proj.dtype, device=proj.device)
        npt = meta.num_prefill_tokens
        if npt:
            ops.gqa_attention_prefill(
                q[:npt], k_cache, v_cache, meta.prefill_block_tables,
                meta.prefill_query_start_loc, meta.prefill_seq_lens, self.scale,
                meta.max_prefill_query_len, out=out[:npt], window=self.window,
                sink=self.sink)
        if meta.num_decode_seqs:
            ops.gqa_attention_decode(
                q[npt:], k_cache, v_cache, meta.decode_block_tables,
                meta.decode_seq_lens, self.scale, out=out[npt:], window=self.window,
                sink=self.sink)
        if self.gate:
            return ops.sigmoid_gate_mul(out, proj[:, c:].view(t, nh, dv))
        return out.view(t, nh * dv)


class BiasedDenseMLP(nn.Module):
    """down(relu(up h + b_up)^2) + b_down."""

    def __init__(self, width: int, ff: int, dtype: torch.dtype):
        super().__init__()
        if get_tp_world_size() != 1:
            raise ValueError("BiasedDenseMLP is not sharded; run it with one rank")
        self.up = _randn_param((ff, width), dtype, std=width ** -0.5)
        self.up_bias = nn.Parameter(torch.zeros(ff, dtype=dtype), requires_grad=False)
        self.down = _randn_param((width, ff), dtype, std=ff ** -0.5)
        self.down_bias = nn.Parameter(torch.zeros(width, dtype=dtype), requires_grad=False)

    def load(self, up, up_b, down, down_b) -> None:
        for p, t in ((self.up, up), (self.up_bias, up_b), (self.down, down),
                     (self.down_bias, down_b)):
            p.data.copy_(t.to(p.dtype))

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        a = ops.relu2(ops.linear(h, self.up), self.up_bias)
        return ops.linear(a, self.down, self.down_bias)


class RoutedExperts(nn.Module):
    """Mixture of ``experts`` small feed-forwards down(relu(up h)^2) (no
    biases) and ``identity`` experts that return their input.

    Router: z = W_r h in f32, s = softmax(z) over all experts + identity; the
    ``top`` largest s + correction are chosen; weights = their s, divided by
    their sum (+ 1e-20).  Returns (y, identity weight [T] f32): y is the
    weighted sum of the chosen real experts, the identity share is left to the
    caller's residual kernel (h times the returned per-row weight).

    Two ways to run the experts, chosen by shape at construction:

    - stacked: one product with all experts' up-projections stacked
      [E * ff, width], the squared relu times the row's weight of the column's
      expert (0 where the expert was not chosen), one product with the
      down-projections stacked along the contraction axis [width, E * ff] —
      the zeros make the unchosen experts vanish exactly.  Any size, f32 or
      bf16, no sorting, shape-static; costs E / top of the chosen experts'
      multiply-adds, so it is the path for few or small experts.
    - grouped: token-expert pairs sorted by expert, one grouped product per
      projection over the expert segments (bf16, sizes in multiples of 128)."""

    def __init__(self, width: int, *, experts: int, identity: int, top: int, ff: int,
                 dtype: torch.dtype, grouped: Optional[bool] = None):
        super().__init__()
        if get_tp_world_size() != 1:
            raise ValueError("RoutedExperts is not sharded; run it with one rank")
        if not 1 <= top <= experts + identity:
            raise ValueError("top must lie between 1 and the number of router outputs")
        self.width, self.experts, self.identity, self.top, self.ff = width, experts, identity, top, ff
        self.dtype = dtype
        fits = dtype == torch.bfloat16 and ff % 128 == 0 and width % 128 == 0
        self.grouped = (fits and experts > 2 * top) if grouped is None else bool(grouped)
        if self.grouped and not fits:
            raise ValueError("grouped experts need bf16 and sizes in multiples of 128")
        self.router = nn.Parameter(
            torch.empty(experts + identity, width, dtype=torch.float32).normal_(0.0, width ** -0.5),
            requires_grad=False)
        self.correction = _f32_param(experts + identity)
        self.up = _randn_param((experts, ff, width), dtype, std=width ** -0.5)
        if self.grouped:
            self.down = _randn_param((experts, width, ff), dtype, std=ff ** -0.5)
        else:
            self.down = _randn_param((width, experts * ff), dtype, std=ff ** -0.5)

    def load(self, router, correction, ups: list, downs: list) -> None:
        self.router.data.copy_(router.float())
        self.correction.data.copy_(correction.float())
        for e, (u, d) in enumerate(zip(ups, downs)):
            self.up.data[e].copy_(u.to(self.dtype))
            if self.grouped:
                self.down.data[e].copy_(d.to(self.dtype))
            else:
                self.down.data[:, e * self.ff:(e + 1) * self.ff].copy_(d.to(self.dtype))

    def forward(self, h: torch.Tensor):
        z = torch.nn.functional.linear(h.float(), self.router)
        dense, ident, ids, w = ops.moe_route(z, self.correction, self.top, self.experts)
        if not self.grouped:
            u = ops.linear(h, self.up.view(self.experts * self.ff, self.width))
            return ops.linear(ops.relu2(u, None, dense), self.down), ident
        ne = self.experts
        # pairs grouped by expert (identity experts get no row)
        xs, pos, seg = ops.moe_sort(ids, ne, h)
        a = ops.moe_gemm(xs, self.up, seg, gated=False, act="relu2")
        ye = ops.moe_gemm(a, self.down, seg, gated=False)
        return ops.moe_combine(ye, pos, ids, w, ne), ident


# ---------------------------------------------------------------------------
# Token shift, differential attention with a chunk mask, HGRN2, sigmoid-routed
# gated experts.
# ---------------------------------------------------------------------------


class TokenShift(nn.Module):
    """h_t + (h_(t-1) - h_t) * w per channel, h the f32 stream as it is before
    the blend; the row before position 0 is zero.  The last row of every
    portion is kept per sequence (f32 [width]) so that portions of any size
    continue where the previous one ended."""

    def __init__(self, width: int, dtype: torch.dtype):
        super().__init__()
        self.width, self.dtype = width, dtype
        self.weight = _f32_param(width)

    def state_shape(self) -> tuple:
        return ("slot", (self.width,), torch.float32)

    def forward(self, x: torch.Tensor, state: torch.Tensor, meta: AttnMetadata) -> torch.Tensor:
        return ops.token_shift_state(x, self.weight, state, meta.seq_start_loc,
                                     meta.seq_lens, meta.state_slots, self.dtype)


def stepped_rotary_frequencies(base: float, dims: int,
                               scaling: Optional[dict] = None) -> list:
    """Frequencies of the dims/2 rotated pairs, f_i = base^(-2i/dims).

    ``scaling`` = {factor, low, high, original}: with the wavelength l = 2 pi /
    f, pairs with l < original/high keep f, pairs with l > original/low turn
    ``factor`` times slower, and between the two f is blended with s =
    (original/l - low) / (high - low): (1 - s) f / factor + s f.  float64;
    callers round once to f32."""
    import math

    freqs = [float(base) ** (-2.0 * i / dims) for i in range(dims // 2)]
    if not scaling:
        return freqs
    factor, low, high = float(scaling["factor"]), float(scaling["low"]), float(scaling["high"])
    orig = float(scaling["original"])
    out = []
    for f in freqs:
        wave = 2.0 * math.pi / f
        if wave < orig / high:
            out.append(f)
        elif wave > orig / low:
            out.append(f / factor)
        else:
            s = (orig / wave - low) / (high - low)
            out.append((1.0 - s) * f / factor + s * f)
    return out


class DiffAttention(_Mixer):
    """Differential grouped-query attention.

    Every query head has two maps (two queries of ``dim`` each) and every
    key/value head two keys and one value: each map is a causal softmax
    attention of its own over the same values, a_1 and a_2, and the head's
    output is (a_1 - lam a_2) / rms(a_1 - lam a_2) * (1 - diff) with lam =
    exp(lq1 . lk1) - exp(lq2 . lk2) + diff, one number for the layer.
    Queries and keys are RMS-normed per head and map (one weight for all of
    them), then their first ``rot_dims`` dims are rotated (dim i with i +
    rot_dims/2).  score = q . k * scale; with ``chunk`` > 0 position i sees j
    <= i only inside its own chunk of that many positions.  Head h's output
    is multiplied by sigmoid(W_g h)_h.

    Projected rows: [q map 1 | q map 2 | k map 1 | k map 2 | v | gate] — the
    maps are laid out as 2H query heads over 2G key heads, so that the usual
    grouped-query rule (query head / (H / G)) finds the right key, and key
    head g reads value head g mod G."""

    def __init__(self, width: int, *, heads: int, kv_heads: int, dim: int, vdim: int,
                 scale: float, diff: float, eps: float, chunk: int = 0,
                 rot_base: float = 10000.0, rot_dims: int = 0,
                 rot_scaling: Optional[dict] = None, head_gate: bool = True,
                 own_in: bool = True, dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        if heads % kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        if rot_dims % 2 or rot_dims > dim:
            raise ValueError("rot_dims must be even and at most dim")
        self.heads, self.kv_heads, self.dim, self.vdim = heads, kv_heads, dim, vdim
        self.scale, self.diff, self.eps, self.chunk = scale, diff, eps, chunk
        self.rot_dims, self.head_gate = rot_dims, head_gate
        rows = 2 * heads * dim + 2 * kv_heads * dim + kv_heads * vdim + (heads if head_gate else 0)
        # zero rows behind the gate keep every projected row 16-byte aligned,
        # which the vector kernels ask for
        self.pad_rows = -rows % 8
        self.in_rows = rows + self.pad_rows
        self.out_rows = heads * vdim
        self._alloc(width, own_in, dtype)
        self.q_norm = _f32_param(dim, fill=1.0)
        self.k_norm = _f32_param(dim, fill=1.0)
        self.lam = diff
        freqs = stepped_rotary_frequencies(rot_base, max(rot_dims, 2), rot_scaling)
        self.register_buffer(
            "inv_freq", torch.tensor(freqs, dtype=torch.float64).to(torch.float32),
            persistent=False)

    def load_in(self, weight, bias, t) -> None:
        nh, ng, d = self.heads, self.kv_heads, self.dim
        # checkpoint rows are head by head [map 1, map 2]; here map by map
        q = t["q"].view(nh, 2, d, -1).transpose(0, 1).reshape(2 * nh * d, -1)
        k = t["k"].view(ng, 2, d, -1).transpose(0, 1).reshape(2 * ng * d, -1)
        off = 0
        for w in [q, k, t["v"]] + ([t["g"]] if self.head_gate else []):
            weight[off:off + w.shape[0]].copy_(w.to(weight.dtype))
            off += w.shape[0]
        if off != self.in_rows - self.pad_rows:
            raise ValueError("projection tensors do not add up to the mixer's rows")
        weight[off:].zero_()

    def load_rest(self, t) -> None:
        import math

        self.q_norm.data.copy_(t["q.norm"].float())
        self.k_norm.data.copy_(t["k.norm"].float())
        dot = lambda a, b: float((t[a].double() * t[b].double()).sum())
        self.lam = math.exp(dot("lq1", "lk1")) - math.exp(dot("lq2", "lk2")) + self.diff

    def cache_shapes(self, block_size: int) -> list:
        return [("paged", (block_size, 2 * self.kv_heads, self.dim), self.dtype),
                ("paged", (block_size, self.kv_heads, self.vdim), self.dtype)]

    def mix(self, proj, positions, cache, meta: AttnMetadata) -> torch.Tensor:
        t = proj.shape[0]
        nh, ng, d, dv = self.heads, self.kv_heads, self.dim, self.vdim
        a = 2 * nh * d
        b = a + 2 * ng * d
        c = b + ng * dv
        k_cache, v_cache = cache
        q = ops.qk_norm_rope_cache_write(
            proj[:, :a].view(t, 2 * nh, d), proj[:, a:b].view(t, 2 * ng, d),
            proj[:, b:c].view(t, ng, dv), self.q_norm, self.k_norm, self.eps, positions,
            self.inv_freq, self.rot_dims, k_cache, v_cache, meta.slot_mapping)
        maps = torch.empty((t, 2 * nh, dv), dtype=torch.float32, device=proj.device)
        npt = meta.num_prefill_tokens
        if npt:
            ops.chunk_attention_prefill(
                q[:npt], k_cache, v_cache, meta.prefill_block_tables,
                meta.prefill_query_start_loc, meta.prefill_seq_lens, self.scale,
                meta.max_prefill_query_len, self.chunk, out=maps[:npt])
        if meta.num_decode_seqs:
            ops.chunk_attention_decode(
                q[npt:], k_cache, v_cache, meta.decode_block_tables,
                meta.decode_seq_lens, self.scale, self.chunk, out=maps[npt:])
        return ops.diff_combine(maps.view(t, 2, nh, dv), self.lam, 1.0 - self.diff, self.eps,
                                proj[:, c:c + nh] if self.head_gate else None, self.dtype)


class HGRN2Mixer(_Mixer):
    """Gated linear recurrence with a matrix state per head.  q = silu(W_q h),
    v = W_v h, forget gate per head and channel g = l + (1 - l) sigmoid(W_f h +
    b) with the lower bound l a weight; S_t = diag(g_t) S_(t-1) + (1 - g_t)
    v_t^T, o_t = S_t^T q_t (no key: 1 - g plays its part); each head's o is
    RMS-normed over vdim with one weight for all heads.  Projected rows:
    [q | f | v]."""

    def __init__(self, width: int, *, heads: int, dim: int, vdim: int, eps: float,
                 own_in: bool = True, dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        self.heads, self.dim, self.vdim, self.eps = heads, dim, vdim, eps
        self.in_rows = 2 * heads * dim + heads * vdim
        self.out_rows = heads * vdim
        self._alloc(width, own_in, dtype)
        self.f_bias = _f32_param(heads * dim)
        self.lower = _f32_param(heads * dim)
        self.norm = _f32_param(heads * vdim, fill=1.0)   # the head weight, repeated

    def load_in(self, weight, bias, t) -> None:
        off = 0
        for name in ("q", "f", "v"):
            n = t[name].shape[0]
            weight[off:off + n].copy_(t[name].to(weight.dtype))
            off += n
        if off != self.in_rows:
            raise ValueError("projection tensors do not add up to the mixer's rows")

    def load_rest(self, t) -> None:
        self.f_bias.data.copy_(t["f.b"].float())
        self.lower.data.copy_(t["lower"].float())
        self.norm.data.copy_(t["norm"].float().repeat(self.heads))

    def cache_shapes(self, block_size: int) -> list:
        return [("slot", (self.heads, self.vdim, self.dim), torch.float32)]

    def mix(self, proj, positions, cache, meta: AttnMetadata) -> torch.Tensor:
        t, nh, d, dv = proj.shape[0], self.heads, self.dim, self.vdim
        a = nh * d
        o = ops.hgrn2_scan(proj[:, :a].view(t, nh, d), proj[:, a:2 * a].view(t, nh, d),
                           proj[:, 2 * a:].view(t, nh, dv), self.f_bias, self.lower,
                           cache[0], meta.seq_start_loc, meta.seq_lens, meta.state_slots)
        return ops.group_rms_norm(o, self.norm, nh, self.eps, self.dtype)


class GatedRoutedExperts(nn.Module):
    """Mixture of ``experts`` small feed-forwards down(silu(gate x) * (up x))
    without biases.  Router: z = W_r h in f32, s = sigmoid(z); the ``top``
    largest s are chosen and weigh their experts as they are (no
    renormalising).  The weight multiplies the expert's *input*: y = sum
    expert(s_e h).

    Without biases gate (s h) = s (gate h), so the weight is applied to the
    projected rows.  Two ways to run the experts, chosen by shape:

    - stacked: one product with every expert's [gate ; up] rows stacked
      [E * 2 ff, width], silu(s g) * (s u) with s = 0 for unchosen experts (they
      vanish exactly), one product with the down-projections stacked along the
      contraction axis.  Any size, f32 or bf16, shape-static.
    - grouped: token-expert pairs grouped by expert, their rows multiplied by
      s, one grouped gated product and one grouped down-projection over the
      expert segments (bf16, sizes in multiples of 128), gather-sum."""

    def __init__(self, width: int, *, experts: int, top: int, ff: int,
                 dtype: torch.dtype, grouped: Optional[bool] = None):
        super().__init__()
        if get_tp_world_size() != 1:
            raise ValueError("GatedRoutedExperts is not sharded; run it with one rank")
        if not 1 <= top <= experts:
            raise ValueError("top must lie between 1 and the number of experts")
        self.width, self.experts, self.top, self.ff = width, experts, top, ff
        self.dtype = dtype
        fits = dtype == torch.bfloat16 and ff % 128 == 0 and width % 128 == 0
        self.grouped = (fits and experts > 2 * top) if grouped is None else bool(grouped)
        if self.grouped and not fits:
            raise ValueError("grouped experts need bf16 and sizes in multiples of 128")
        self.router = nn.Parameter(
            torch.empty(experts, width, dtype=torch.float32).normal_(0.0, width ** -0.5),
            requires_grad=False)
        # per expert: ff gate rows, then ff up rows
        self.gate_up = _randn_param((experts, 2 * ff, width), dtype, std=width ** -0.5)
        if self.grouped:
            self.down = _randn_param((experts, width, ff), dtype, std=ff ** -0.5)
        else:
            self.down = _randn_param((width, experts * ff), dtype, std=ff ** -0.5)

    def load(self, router, gates: list, ups: list, downs: list) -> None:
        self.router.data.copy_(router.float())
        ff = self.ff
        for e, (g, u, d) in enumerate(zip(gates, ups, downs)):
            self.gate_up.data[e, :ff].copy_(g.to(self.dtype))
            self.gate_up.data[e, ff:].copy_(u.to(self.dtype))
            if self.grouped:
                self.down.data[e].copy_(d.to(self.dtype))
            else:
                self.down.data[:, e * ff:(e + 1) * ff].copy_(d.to(self.dtype))

    def forward(self, h: torch.Tensor, router_in: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``router_in``: the f32 rows h was rounded from, when the caller has
        them; the router then reads those instead of the rounded copy."""
        z = torch.nn.functional.linear(h.float() if router_in is None else router_in,
                                       self.router)
        dense, ids, w = ops.moe_route_sigmoid(z, self.top)
        ne = self.experts
        if not self.grouped:
            gu = ops.linear(h, self.gate_up.view(ne * 2 * self.ff, self.width))
            return ops.linear(ops.silu_mul_scaled(gu, dense), self.down)
        xs, pos, seg = ops.moe_sort(ids, ne, h, row_scale=w)
        a = ops.moe_gemm(xs, self.gate_up, seg, gated=True)
        ye = ops.moe_gemm(a, self.down, seg, gated=False)
        return ops.moe_combine(ye, pos, ids, torch.ones_like(w), ne)
