"""Plain-PyTorch reference implementations of every custom op.

These are the CPU execution path (protocol tests run the full engine on CPU,
like the reference's CPU-build CI — SURVEY.md §4) and the numerics oracle the
GPU kernels are tested against (fp32 upcast).
"""

from __future__ import annotations

import torch


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    xf = x.float()
    var = xf.pow(2).mean(dim=-1, keepdim=True)
    out = xf * torch.rsqrt(var + eps)
    return (out * weight.float()).to(x.dtype)


def fused_add_rms_norm(
    x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float
) -> tuple[torch.Tensor, torch.Tensor]:
    """Returns (normed, new_residual) where new_residual = x + residual."""
    summed = (x.float() + residual.float()).to(x.dtype)
    return rms_norm(summed, weight, eps), summed


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    d = x.shape[-1] // 2
    a, b = x[..., :d], x[..., d:]
    return (torch.nn.functional.silu(a.float()) * b.float()).to(x.dtype)


def make_cos_sin_cache(
    head_dim: int, max_len: int, theta: float, dtype: torch.dtype,
    scaling: dict | None = None,
) -> torch.Tensor:
    """[max_len, head_dim] cache: first half cos, second half sin (f32)."""
    rot = head_dim
    inv_freq = 1.0 / (theta ** (torch.arange(0, rot, 2, dtype=torch.float64) / rot))
    if scaling and scaling.get("rope_type") == "llama3":
        # llama-3.1-style frequency rescaling
        factor = scaling["factor"]
        lo = scaling.get("low_freq_factor", 1.0)
        hi = scaling.get("high_freq_factor", 4.0)
        orig = scaling.get("original_max_position_embeddings", 8192)
        wavelen = 2 * torch.pi / inv_freq
        ratio = orig / wavelen
        smooth = ((ratio - lo) / (hi - lo)).clamp(0, 1)
        inv_freq = torch.where(
            wavelen > orig / lo,
            torch.where(wavelen < orig / hi, inv_freq, inv_freq / factor),
            inv_freq * ((1 - smooth) / factor + smooth),
        )
    t = torch.arange(max_len, dtype=torch.float64)
    freqs = torch.outer(t, inv_freq)
    return torch.cat([freqs.cos(), freqs.sin()], dim=-1).float()


def rotary_embedding(
    positions: torch.Tensor,  # [T]
    q: torch.Tensor,          # [T, num_heads * head_dim]
    k: torch.Tensor,          # [T, num_kv_heads * head_dim]
    head_dim: int,
    cos_sin_cache: torch.Tensor,  # [max_len, head_dim] f32
) -> tuple[torch.Tensor, torch.Tensor]:
    """NeoX-style (rotate halves) rotary embedding, out-of-place reference."""
    half = head_dim // 2
    cs = cos_sin_cache[positions]          # [T, head_dim]
    cos = cs[:, :half].unsqueeze(1)        # [T, 1, half]
    sin = cs[:, half:].unsqueeze(1)

    def rot(x: torch.Tensor) -> torch.Tensor:
        t = x.shape[0]
        xs = x.view(t, -1, head_dim).float()
        x1, x2 = xs[..., :half], xs[..., half:]
        o1 = x1 * cos - x2 * sin
        o2 = x2 * cos + x1 * sin
        return torch.cat([o1, o2], dim=-1).to(x.dtype).view(t, -1)

    return rot(q), rot(k)


def reshape_and_cache(
    k: torch.Tensor,  # [T, num_kv_heads, head_dim]
    v: torch.Tensor,
    k_cache: torch.Tensor,  # [num_blocks, block_size, num_kv_heads, head_dim]
    v_cache: torch.Tensor,
    slot_mapping: torch.Tensor,  # [T] int64 (flat slot = block*block_size + off)
) -> None:
    bs = k_cache.shape[1]
    blocks = torch.div(slot_mapping, bs, rounding_mode="floor")
    offs = slot_mapping % bs
    k_cache[blocks, offs] = k.to(k_cache.dtype)
    v_cache[blocks, offs] = v.to(v_cache.dtype)


def _gather_kv(
    k_cache: torch.Tensor, v_cache: torch.Tensor,
    block_table: torch.Tensor, seq_len: int,
) -> tuple[torch.Tensor, torch.Tensor]:
    bs = k_cache.shape[1]
    nb = (seq_len + bs - 1) // bs
    k = k_cache[block_table[:nb]].reshape(-1, *k_cache.shape[2:])[:seq_len]
    v = v_cache[block_table[:nb]].reshape(-1, *v_cache.shape[2:])[:seq_len]
    return k, v


def paged_attention(
    q: torch.Tensor,            # [T, num_heads, head_dim]
    k_cache: torch.Tensor,      # [num_blocks, block_size, num_kv_heads, head_dim]
    v_cache: torch.Tensor,
    block_tables: torch.Tensor,  # [num_seqs, max_blocks]
    query_start_loc: torch.Tensor,  # [num_seqs + 1] (cpu)
    seq_lens: torch.Tensor,         # [num_seqs] total context per seq (cpu)
    scale: float,
    window: int = 0,
    sink: float | None = None,
) -> torch.Tensor:
    """Causal paged attention over queries that are the *tail* of each
    sequence (covers prefill chunks and single-token decode uniformly).
    ``window`` > 0: a query at position i sees keys j with 0 <= i - j < window.
    ``sink``: the softmax denominator also holds exp(sink) (no key, no value)."""
    num_heads = q.shape[1]
    num_kv_heads = k_cache.shape[2]
    group = num_heads // num_kv_heads
    # the value size may differ from the query/key size
    out = torch.empty((q.shape[0], num_heads, v_cache.shape[-1]), dtype=q.dtype,
                      device=q.device)
    qs = query_start_loc.tolist()
    lens = seq_lens.tolist()
    for i in range(len(lens)):
        s, e = qs[i], qs[i + 1]
        q_len = e - s
        seq_len = lens[i]
        if q_len == 0 or seq_len == 0:
            out[s:e] = 0
            continue
        k, v = _gather_kv(k_cache, v_cache, block_tables[i], seq_len)
        qf = q[s:e].float()                       # [q, H, d]
        kf = k.float().repeat_interleave(group, dim=1)  # [S, H, d]
        vf = v.float().repeat_interleave(group, dim=1)
        scores = torch.einsum("qhd,shd->hqs", qf, kf) * scale
        # causal: query position j (global seq_len - q_len + j) sees keys <= it
        kpos = torch.arange(seq_len, device=q.device)
        qpos = torch.arange(seq_len - q_len, seq_len, device=q.device)
        mask = kpos[None, :] > qpos[:, None]
        if window > 0:
            mask = mask | (qpos[:, None] - kpos[None, :] >= window)
        scores.masked_fill_(mask.unsqueeze(0), float("-inf"))
        if sink is None:
            probs = torch.softmax(scores, dim=-1)
        else:
            m = scores.max(dim=-1, keepdim=True).values.clamp(min=float(sink))
            probs = torch.exp(scores - m)
            probs = probs / (probs.sum(dim=-1, keepdim=True) + torch.exp(float(sink) - m))
        out[s:e] = torch.einsum("hqs,shd->qhd", probs, vf).to(q.dtype)
    return out


def topk_softmax(gate_logits: torch.Tensor, top_k: int) -> tuple[torch.Tensor, torch.Tensor]:
    """MoE router: softmax over experts then top-k, renormalized."""
    probs = torch.softmax(gate_logits.float(), dim=-1)
    weights, ids = torch.topk(probs, top_k, dim=-1)
    weights = weights / weights.sum(dim=-1, keepdim=True)
    return weights, ids


# ---------------------------------------------------------------------------
# f32 residual-stream ops, short causal convolution with per-sequence state,
# windowed latent attention with sinks (the `_C_seq` and `_C_lat` kernel sets)
# ---------------------------------------------------------------------------


def gelu_tanh(x: torch.Tensor, mul: torch.Tensor | None = None) -> torch.Tensor:
    z = x.float()
    y = 0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z * z * z)))
    if mul is not None:
        y = y * mul.float()
    return y.to(x.dtype)


def embedding_scaled(ids: torch.Tensor, table: torch.Tensor, scale: float) -> torch.Tensor:
    return table[ids].float() * scale


def rms_norm_stream(x: torch.Tensor, weight: torch.Tensor, eps: float,
                    weight_offset: float, out_dtype: torch.dtype) -> torch.Tensor:
    xf = x.float()
    r = torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + eps)
    return (xf * r * (weight.float() + weight_offset)).to(out_dtype)


def stream_add(x: torch.Tensor, a: torch.Tensor, b: torch.Tensor | None,
               mult: float, cast_dtype: torch.dtype | None) -> torch.Tensor | None:
    s = a.float() if b is None else a.float() + b.float()
    x.add_(s, alpha=mult)
    return x.to(cast_dtype) if cast_dtype is not None else None


def stream_add_rms_norm(x: torch.Tensor, y: torch.Tensor, weight: torch.Tensor,
                        eps: float, mult: float,
                        layer_scale: torch.Tensor | None = None) -> None:
    yf = y.float()
    r = torch.rsqrt(yf.pow(2).mean(dim=-1, keepdim=True) + eps)
    n = yf * r * weight.float()
    if layer_scale is not None:
        n = n * layer_scale.float()
    x.add_(n, alpha=mult)


def softcap(logits: torch.Tensor, cap: float) -> torch.Tensor:
    lf = logits.float()
    return cap * torch.tanh(lf / cap)


def causal_conv_state(
    h: torch.Tensor,            # [T, W] (rows may be strided)
    weight: torch.Tensor,       # [W, taps]
    state: torch.Tensor,        # [slots, taps-1, W]
    seq_start_loc: torch.Tensor,  # [S+1] rows of each sequence's new tokens
    seq_lens: torch.Tensor,       # [S] tokens of the sequence incl. the new ones
    state_slots: torch.Tensor,    # [S]
    add_input: bool,
    bias: torch.Tensor | None = None,   # [W] f32
    act: str | None = None,             # None | "silu"
) -> torch.Tensor:
    """out_t = (h_t if add_input) + sum_j w[:, j] * h_(t - taps + 1 + j) per
    sequence, inputs before the step's rows come from ``state`` (the last
    taps-1 inputs of the sequence), inputs before the sequence are zero;
    ``state`` is then advanced past the new rows."""
    taps = weight.shape[1]
    out = torch.empty(h.shape, dtype=h.dtype, device=h.device)
    loc = seq_start_loc.tolist()
    lens = seq_lens.tolist()
    slots = state_slots.tolist()
    wf = weight.float()
    for i in range(len(lens)):
        a, b = loc[i], loc[i + 1]
        n = b - a
        if n == 0:
            continue
        if slots[i] < 0:
            out[a:b] = 0
            continue
        start = lens[i] - n
        hist = state[slots[i]].float() if taps > 1 else h.new_zeros((0, h.shape[1]), dtype=torch.float32)
        if taps > 1:
            # state row j is position start - (taps-1) + j; negative => zero
            valid = (torch.arange(taps - 1) + start - (taps - 1)) >= 0
            hist = hist * valid.to(hist.dtype).unsqueeze(1).to(hist.device)
        ext = torch.cat([hist, h[a:b].float()], dim=0)     # [taps-1+n, W]
        acc = h[a:b].float().clone() if add_input else torch.zeros_like(ext[taps - 1:])
        for j in range(taps):
            acc = acc + wf[:, j] * ext[j:j + n]
        if bias is not None:
            acc = acc + bias.float()
        if act == "silu":
            acc = acc * torch.sigmoid(acc)
        out[a:b] = acc.to(h.dtype)
        if taps > 1:
            state[slots[i]] = ext[n:].to(state.dtype)
    return out


def rope_partial(x: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor,
                 offset: int, rot_dims: int, interleaved: bool = False,
                 mag: float = 1.0) -> None:
    """In place: dims [offset, offset+rot_dims) of the last axis of x [T, H, D]
    are rotated, dim i paired with i + rot_dims/2 (or, ``interleaved``, dim 2i
    with 2i+1), angle = position * inv_freq[i] in f32; cos and sin are
    multiplied by ``mag``."""
    half = rot_dims // 2
    ang = positions.to(torch.float32).unsqueeze(1) * inv_freq.float().unsqueeze(0)
    cos, sin = ang.cos().unsqueeze(1), ang.sin().unsqueeze(1)
    if mag != 1.0:
        cos, sin = cos * mag, sin * mag
    if interleaved:
        ia = slice(offset, offset + rot_dims, 2)
        ib = slice(offset + 1, offset + rot_dims, 2)
    else:
        ia = slice(offset, offset + half)
        ib = slice(offset + half, offset + rot_dims)
    u = x[..., ia].float()
    v = x[..., ib].float()
    a = (u * cos - v * sin).to(x.dtype)   # both halves before either store:
    b = (v * cos + u * sin).to(x.dtype)   # for f32 x, u and v alias x
    x[..., ia] = a
    x[..., ib] = b


def latent_kv_write(
    dkv: torch.Tensor,          # [T, rank + rot]
    norm_weight: torch.Tensor,  # [rank]
    eps: float,
    positions: torch.Tensor,
    inv_freq: torch.Tensor,     # [rot_dims/2] f32
    rot_dims: int,
    cache: torch.Tensor,        # [blocks, block_size, rank + rot]
    slot_mapping: torch.Tensor,
    interleaved: bool = False,
    mag: float = 1.0,
) -> None:
    rank = norm_weight.shape[0]
    c = dkv[:, :rank].float()
    c = c * torch.rsqrt(c.pow(2).mean(dim=-1, keepdim=True) + eps) * norm_weight.float()
    kr = dkv[:, rank:].float().unsqueeze(1).clone()
    rope_partial(kr, positions, inv_freq, 0, rot_dims, interleaved, mag)
    row = torch.cat([c, kr.squeeze(1)], dim=-1).to(cache.dtype)
    bs = cache.shape[1]
    ok = slot_mapping >= 0
    sm = slot_mapping[ok]
    cache[torch.div(sm, bs, rounding_mode="floor"), sm % bs] = row[ok]


def latent_attention(
    q_lat: torch.Tensor,        # [T, H, rank]  (queries folded into latent space)
    q_rot: torch.Tensor,        # [T, H, rot]
    cache: torch.Tensor,        # [blocks, block_size, rank + rot]
    block_tables: torch.Tensor,
    query_start_loc: torch.Tensor,
    seq_lens: torch.Tensor,
    scale: float,
    window: int,                # 0 = unbounded causal
    sinks: torch.Tensor | None,  # [H] f32
) -> torch.Tensor:
    """Multi-query attention of every head over one shared latent row per
    token: score = (q_lat . c + q_rot . k_rot) * scale, softmax whose
    denominator also holds exp(sink_h), value = c.  Queries are the tail of
    each sequence."""
    t, nh, rank = q_lat.shape
    out = torch.zeros((t, nh, rank), dtype=q_lat.dtype, device=q_lat.device)
    qs = query_start_loc.tolist()
    lens = seq_lens.tolist()
    bs = cache.shape[1]
    for i in range(len(lens)):
        s, e = qs[i], qs[i + 1]
        n, sl = e - s, lens[i]
        if n == 0 or sl == 0:
            continue
        nb = (sl + bs - 1) // bs
        kv = cache[block_tables[i, :nb].long()].reshape(-1, cache.shape[-1])[:sl].float()
        q = torch.cat([q_lat[s:e].float(), q_rot[s:e].float()], dim=-1)
        sc = torch.einsum("qhd,sd->hqs", q, kv) * scale
        kpos = torch.arange(sl)
        qpos = torch.arange(sl - n, sl)
        dist = qpos[:, None] - kpos[None, :]
        bad = dist < 0
        if window > 0:
            bad = bad | (dist >= window)
        sc = sc.masked_fill(bad.unsqueeze(0).to(sc.device), float("-inf"))
        m = sc.max(dim=-1).values
        if sinks is not None:
            m = torch.maximum(m, sinks.float().view(-1, 1))
        p = torch.exp(sc - m.unsqueeze(-1))
        den = p.sum(dim=-1)
        if sinks is not None:
            den = den + torch.exp(sinks.float().view(-1, 1) - m)
        p = p / den.unsqueeze(-1)
        out[s:e] = torch.einsum("hqs,sd->qhd", p, kv[:, :rank]).to(out.dtype)
    return out


# ---------------------------------------------------------------------------
# Layer norm of an f32 stream, per-head query/key RMS norm with a query
# temperature, recurrent mixers with per-sequence f32 state (matrix-state
# scans of the SSD and mLSTM kind, the gated linear recurrent unit)
# ---------------------------------------------------------------------------


def _layer_norm_f32(xf: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    mu = xf.mean(dim=-1, keepdim=True)
    d = xf - mu
    var = (d * d).mean(dim=-1, keepdim=True)
    return d * torch.rsqrt(var + eps) * weight.float()


def layer_norm_stream(x: torch.Tensor, weight: torch.Tensor, eps: float,
                      out_dtype: torch.dtype) -> torch.Tensor:
    """Bias-free layer norm of an f32 stream into the compute dtype."""
    return _layer_norm_f32(x.float(), weight, eps).to(out_dtype)


def stream_add_layer_norm(x: torch.Tensor, a: torch.Tensor, b: torch.Tensor | None,
                          scale_a: float, scale_b: float, weight: torch.Tensor,
                          layer_scale: torch.Tensor | None, eps: float) -> None:
    """x (f32, in place) += LN(scale_a * a + scale_b * b) * weight * layer_scale."""
    y = a.float() * scale_a
    if b is not None:
        y = y + b.float() * scale_b
    y = _layer_norm_f32(y, weight, eps)
    if layer_scale is not None:
        y = y * layer_scale.float()
    x.add_(y)


def stream_add_vec(x: torch.Tensor, other: torch.Tensor | None, vec: torch.Tensor) -> None:
    """x (f32, in place) += other + vec (vec broadcast over rows)."""
    if other is not None:
        x.add_(other)
    x.add_(vec.float())


def qk_norm_cache_write(
    q: torch.Tensor,            # [T, H, dim]  (may be a strided view)
    k: torch.Tensor,            # [T, G, dim]
    v: torch.Tensor,            # [T, G, vdim]
    q_weight: torch.Tensor,     # [dim] f32
    k_weight: torch.Tensor,     # [dim] f32
    eps: float,
    positions: torch.Tensor,    # [T] int64
    temp_coef: float,
    temp_every: int,            # 0 = no query temperature
    k_cache: torch.Tensor,      # [blocks, block, G, dim]
    v_cache: torch.Tensor,      # [blocks, block, G, vdim]
    slot_mapping: torch.Tensor,
) -> torch.Tensor:
    """Per-head RMS norm of queries and keys (f32 statistics, plain weight);
    queries are then multiplied by 1 + coef * ln(floor((p + 1) / every) + 1);
    normed keys and the values go to the paged cache.  Returns the queries
    [T, H, dim] (contiguous)."""
    qf = q.float()
    qf = qf * torch.rsqrt(qf.pow(2).mean(dim=-1, keepdim=True) + eps) * q_weight.float()
    if temp_every > 0:
        p = positions.to(torch.float32)
        temp = 1.0 + temp_coef * torch.log(torch.floor((p + 1.0) / temp_every) + 1.0)
        qf = qf * temp.view(-1, 1, 1)
    kf = k.float()
    kf = kf * torch.rsqrt(kf.pow(2).mean(dim=-1, keepdim=True) + eps) * k_weight.float()
    ok = slot_mapping >= 0
    sm = slot_mapping[ok]
    bs = k_cache.shape[1]
    blk = torch.div(sm, bs, rounding_mode="floor")
    k_cache[blk, sm % bs] = kf[ok].to(k_cache.dtype)
    v_cache[blk, sm % bs] = v[ok].to(v_cache.dtype)
    return qf.to(q.dtype).contiguous()


def _softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.nn.functional.softplus(z, beta=1.0, threshold=30.0)


def _seq_iter(seq_start_loc, seq_lens, state_slots):
    loc = seq_start_loc.tolist()
    lens = seq_lens.tolist()
    slots = state_slots.tolist()
    for i in range(len(lens)):
        a, b = loc[i], loc[i + 1]
        if b > a:
            yield a, b, lens[i] - (b - a), slots[i]


def ssd_scan(
    xbc: torch.Tensor,          # [T, inner + 2*G*N] after convolution + activation
    dt: torch.Tensor,           # [T, H] raw step sizes (may be a strided view)
    dt_bias: torch.Tensor,      # [H] f32
    a_log: torch.Tensor,        # [H] f32
    d_skip: torch.Tensor,       # [H] f32
    state: torch.Tensor,        # [slots, H, vdim, N] f32
    seq_start_loc, seq_lens, state_slots,
    heads: int, vdim: int, nstate: int, groups: int,
) -> torch.Tensor:
    """S_t = exp(-exp(A_log) * dt_t) S_(t-1) + dt_t * B_t x_t^T, y_t = S_t^T C_t
    + D x_t per head, dt_t = softplus(dt + dt_bias); f32 throughout; a sequence
    that starts in this step starts from S = 0 whatever its slot holds.
    Returns y [T, H*vdim] f32."""
    t = xbc.shape[0]
    inner = heads * vdim
    y = torch.zeros((t, heads, vdim), dtype=torch.float32, device=xbc.device)
    xf = xbc.float()
    dtf = _softplus(dt.float() + dt_bias.float())
    decay = torch.exp(-torch.exp(a_log.float()) * dtf)          # [T, H]
    per = heads // groups
    for a, b, start, slot in _seq_iter(seq_start_loc, seq_lens, state_slots):
        if slot < 0:
            continue
        s = state[slot].clone() if start > 0 else torch.zeros_like(state[slot])
        for i in range(a, b):
            x = xf[i, :inner].view(heads, vdim)
            bm = xf[i, inner:inner + groups * nstate].view(groups, nstate)
            cm = xf[i, inner + groups * nstate:].view(groups, nstate)
            bm = bm.repeat_interleave(per, dim=0)               # [H, N]
            cm = cm.repeat_interleave(per, dim=0)
            s = decay[i].view(heads, 1, 1) * s \
                + x.unsqueeze(2) * (dtf[i].view(heads, 1) * bm).unsqueeze(1)
            y[i] = torch.einsum("hvn,hn->hv", s, cm) + d_skip.float().view(heads, 1) * x
        state[slot] = s
    return y.view(t, inner)


def gated_group_norm(
    y: torch.Tensor,            # [T, C] f32
    gate: torch.Tensor,         # [T, C] compute dtype (may be a strided view)
    weight: torch.Tensor,       # [C] f32
    groups: int,
    eps: float,
    gate_first: bool,
    out_dtype: torch.dtype,
) -> torch.Tensor:
    """gate_first: RMS-norm of y * silu(gate) in ``groups`` equal parts, times
    weight.  Otherwise: RMS-norm of y in parts, times weight, times
    sigmoid(gate)."""
    t, c = y.shape
    yf = y.float()
    gf = gate.float()
    if gate_first:
        yf = yf * (gf * torch.sigmoid(gf))
    yg = yf.view(t, groups, c // groups)
    yg = yg * torch.rsqrt(yg.pow(2).mean(dim=-1, keepdim=True) + eps)
    out = yg.reshape(t, c) * weight.float()
    if not gate_first:
        out = out * torch.sigmoid(gf)
    return out.to(out_dtype)


def rglru_scan(
    u: torch.Tensor,            # [T, W] convolved input branch
    r_pre: torch.Tensor,        # [T, W] recurrence-gate pre-activation (no bias)
    i_pre: torch.Tensor,        # [T, W] input-gate pre-activation (no bias)
    r_bias: torch.Tensor,       # [W] f32
    i_bias: torch.Tensor,       # [W] f32
    lam: torch.Tensor,          # [W] f32
    gate_c: float,              # the constant in log a = -c * r * softplus(lam)
    y_branch: torch.Tensor,     # [T, W] the other branch, multiplied in at the end
    state: torch.Tensor,        # [slots, W] f32
    seq_start_loc, seq_lens, state_slots,
) -> torch.Tensor:
    """S_t = a_t S_(t-1) + sqrt(1 - a_t^2) * i_t * u_t with a_t = exp(-c * r_t *
    softplus(lam)); returns S_t * y_t in u's dtype."""
    uf = u.float()
    r = torch.sigmoid(r_pre.float() + r_bias.float())
    g = torch.sigmoid(i_pre.float() + i_bias.float())
    log_a = -gate_c * r * _softplus(lam.float())
    a_ = torch.exp(log_a)
    inp = torch.sqrt(1.0 - a_ * a_) * g * uf
    out = torch.zeros(u.shape, dtype=torch.float32, device=u.device)
    for a, b, start, slot in _seq_iter(seq_start_loc, seq_lens, state_slots):
        if slot < 0:
            continue
        s = state[slot].clone() if start > 0 else torch.zeros_like(state[slot])
        for i in range(a, b):
            s = a_[i] * s + inp[i]
            out[i] = s
        state[slot] = s
    return (out * y_branch.float()).to(u.dtype)


def mlstm_scan(
    q: torch.Tensor,            # [T, H, dim]
    k: torch.Tensor,            # [T, H, dim]
    v: torch.Tensor,            # [T, H, vdim]
    i_pre: torch.Tensor,        # [T, H] input-gate pre-activation (no bias)
    f_pre: torch.Tensor,        # [T, H] forget-gate pre-activation (no bias)
    i_bias: torch.Tensor,       # [H] f32
    f_bias: torch.Tensor,       # [H] f32
    cap: float,
    q_scale: float,
    s_state: torch.Tensor,      # [slots, H, vdim, dim] f32
    n_state: torch.Tensor,      # [slots, H, dim] f32
    m_state: torch.Tensor,      # [slots, H] f32
    seq_start_loc, seq_lens, state_slots,
) -> torch.Tensor:
    """Matrix memory with exponential gates held stable by a running maximum m
    (initialised to 0): i = cap * tanh((i_pre + b) / cap), f =
    logsigmoid(cap * tanh((f_pre + b) / cap)), m_t = max(f + m, i), S_t =
    exp(f + m - m_t) S + exp(i - m_t) k v^T, n_t likewise with k, o = S_t^T q /
    (max(|n_t . q|, exp(-m_t)) + 1e-6).  Returns o [T, H*vdim] f32."""
    t, heads, dim = q.shape
    vdim = v.shape[-1]
    qf = q.float() * q_scale
    kf, vf = k.float(), v.float()
    ig = cap * torch.tanh((i_pre.float() + i_bias.float()) / cap)
    fg = torch.nn.functional.logsigmoid(
        cap * torch.tanh((f_pre.float() + f_bias.float()) / cap))
    o = torch.zeros((t, heads, vdim), dtype=torch.float32, device=q.device)
    for a, b, start, slot in _seq_iter(seq_start_loc, seq_lens, state_slots):
        if slot < 0:
            continue
        if start > 0:
            s, n, m = s_state[slot].clone(), n_state[slot].clone(), m_state[slot].clone()
        else:
            s = torch.zeros_like(s_state[slot])
            n = torch.zeros_like(n_state[slot])
            m = torch.zeros_like(m_state[slot])
        for i in range(a, b):
            m_new = torch.maximum(fg[i] + m, ig[i])
            fd = torch.exp(fg[i] + m - m_new)
            idc = torch.exp(ig[i] - m_new)
            s = fd.view(heads, 1, 1) * s + idc.view(heads, 1, 1) * vf[i].unsqueeze(2) * kf[i].unsqueeze(1)
            n = fd.view(heads, 1) * n + idc.view(heads, 1) * kf[i]
            m = m_new
            den = torch.maximum((n * qf[i]).sum(dim=-1).abs(), torch.exp(-m)) + 1e-6
            o[i] = torch.einsum("hvd,hd->hv", s, qf[i]) / den.view(heads, 1)
        s_state[slot], n_state[slot], m_state[slot] = s, n, m
    return o.view(t, heads * vdim)


# ---------------------------------------------------------------------------
# Two-norm parallel layers, rotated grouped-query attention whose cache is
# written by one op, output gates, squared-relu feed-forwards, routed experts
# with identity experts
# ---------------------------------------------------------------------------


def stream_add_rms_norm_pair(x: torch.Tensor, a: torch.Tensor | None,
                             b: torch.Tensor | None, row_scale: torch.Tensor | None,
                             c: torch.Tensor | None, w1: torch.Tensor | None,
                             w2: torch.Tensor | None, eps: float,
                             out_dtype: torch.dtype):
    """x (f32, in place) += a + b + row_scale[:, None] * c (each optional), then
    two RMS norms of the updated row that share one statistic:
    x / sqrt(mean(x^2) + eps) * w1 and * w2.  Returns (h1, h2), None where the
    weight is None."""
    if a is not None:
        s = a.float()
        if b is not None:
            s = s + b.float()
        if c is not None:
            s = s + row_scale.float().unsqueeze(1) * c.float()
        x.add_(s)
    if w1 is None and w2 is None:
        return None, None
    u = x * torch.rsqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)
    h1 = (u * w1.float()).to(out_dtype) if w1 is not None else None
    h2 = (u * w2.float()).to(out_dtype) if w2 is not None else None
    return h1, h2


def rope_kv_cache_write(q, k, v, positions, inv_freq, rot_dims: int, interleaved: bool,
                        mag: float, k_cache, v_cache, slot_mapping) -> torch.Tensor:
    """Rotate the first ``rot_dims`` dims of every head of q [T, H, dim] and
    k [T, G, dim]; store rotated keys and v [T, G, vdim] (as given) in the paged
    cache (slot < 0: skipped).  Returns contiguous rotated queries."""
    qo = q.clone()
    kr = k.clone()
    if rot_dims:
        rope_partial(qo, positions, inv_freq, 0, rot_dims, interleaved, mag)
        rope_partial(kr, positions, inv_freq, 0, rot_dims, interleaved, mag)
    bs = k_cache.shape[1]
    ok = slot_mapping >= 0
    sm = slot_mapping[ok]
    blk, off = torch.div(sm, bs, rounding_mode="floor"), sm % bs
    k_cache[blk, off] = kr[ok].to(k_cache.dtype)
    v_cache[blk, off] = v[ok].to(v_cache.dtype)
    return qo


def sigmoid_gate_mul(o: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
    """o [T, H, D] (any strides) times sigmoid(gate), gate [T, H, D] (one per
    element) or [T, H] (one per head); f32 sigmoid; returns contiguous
    [T, H * D]."""
    t, h, d = o.shape
    g = torch.sigmoid(gate.float())
    g = g.unsqueeze(-1) if gate.dim() == 2 else g
    return (o.float() * g).to(o.dtype).reshape(t, h * d)


def relu2(x: torch.Tensor, bias: torch.Tensor | None = None,
          col_scale: torch.Tensor | None = None) -> torch.Tensor:
    """relu(x + bias)^2, optionally times col_scale[t, column // (cols / E)]
    (col_scale [T, E] f32: one factor per row and block of columns)."""
    z = x.float()
    if bias is not None:
        z = z + bias.float()
    z = torch.clamp(z, min=0.0)
    z = z * z
    if col_scale is not None:
        e = col_scale.shape[1]
        z = (z.view(z.shape[0], e, -1) * col_scale.float().unsqueeze(-1)).view(z.shape)
    return z.to(x.dtype)


def moe_route(logits: torch.Tensor, correction: torch.Tensor, top: int, num_real: int):
    """Router of a mixture with identity experts.  logits [T, N] f32 over the
    ``num_real`` real experts followed by N - num_real identity experts.
    s = softmax(logits); the ``top`` experts with the largest s + correction
    are chosen (ties: the lower index); weights = s[chosen] / (sum + 1e-20).
    Returns (dense [T, num_real] f32: weight of each real expert or 0,
    identity [T] f32: summed weight of the chosen identity experts,
    ids [T, top] int32, weights [T, top] f32)."""
    s = torch.softmax(logits.float(), dim=-1)
    choice = s + correction.float()
    # stable descending order: ties go to the lower index
    order = torch.sort(choice, dim=-1, descending=True, stable=True).indices[:, :top]
    w = torch.gather(s, 1, order)
    w = w / (w.sum(dim=-1, keepdim=True) + 1e-20)
    full = torch.zeros_like(s).scatter_(1, order, w)
    return (full[:, :num_real].contiguous(), full[:, num_real:].sum(dim=-1),
            order.to(torch.int32), w)


def moe_combine(ye: torch.Tensor, pos: torch.Tensor, ids: torch.Tensor,
                weights: torch.Tensor, num_real: int) -> torch.Tensor:
    """out[t] = sum over k with ids[t, k] < num_real of weights[t, k] *
    ye[pos[t, k]] (ye: expert outputs of the token-expert pairs sorted by
    expert, pos [T, top]: where pair (t, k) went); f32 sums."""
    rows = ye[pos.long().reshape(-1)].float().view(*pos.shape, -1)
    w = torch.where(ids < num_real, weights.float(), torch.zeros_like(weights, dtype=torch.float32))
    rows = torch.where((ids < num_real).unsqueeze(-1), rows, torch.zeros_like(rows))
    return (rows * w.unsqueeze(-1)).sum(dim=1).to(ye.dtype)


def moe_gemm(x: torch.Tensor, w: torch.Tensor, seg_off: torch.Tensor, gated: bool,
             act: str | None = None) -> torch.Tensor:
    """Rows seg_off[e] .. seg_off[e+1] of x times expert e's weight w[e]
    ([2N, K] gated: silu(first half) * second half; else [N, K], optionally
    followed by the squared relu).  Rows past the last segment are zeros."""
    n = w.shape[1] // 2 if gated else w.shape[1]
    out = torch.zeros((x.shape[0], n), dtype=x.dtype, device=x.device)
    off = seg_off.tolist()
    for e in range(w.shape[0]):
        a, b = off[e], off[e + 1]
        if b <= a:
            continue
        y = x[a:b].float() @ w[e].float().T
        if gated:
            y = torch.nn.functional.silu(y[:, :n]) * y[:, n:]
        elif act == "relu2":
            y = torch.clamp(y, min=0.0) ** 2
        out[a:b] = y.to(x.dtype)
    return out


def moe_sort(ids: torch.Tensor, num_real: int, h: torch.Tensor,
             row_scale: torch.Tensor | None = None):
    """Token-expert pairs grouped by expert (stable): gathered rows (times
    row_scale[t, k] f32 when given), each pair's row, segment offsets of the
    real experts."""
    t, top = ids.shape
    flat = ids.reshape(-1).long()
    order = torch.argsort(flat, stable=True)
    pos = torch.empty_like(order)
    pos[order] = torch.arange(t * top, device=ids.device)
    counts = torch.bincount(flat, minlength=num_real)[:num_real]
    seg = torch.zeros(num_real + 1, dtype=torch.int32, device=ids.device)
    seg[1:] = counts.cumsum(0).to(torch.int32)
    xs = h[torch.div(order, top, rounding_mode="floor")]
    if row_scale is not None:
        xs = (xs.float() * row_scale.reshape(-1)[order].float().unsqueeze(1)).to(h.dtype)
    pos = torch.where(flat < num_real, pos, torch.zeros_like(pos))
    return xs, pos.view(t, top).to(torch.int32), seg


# ---------------------------------------------------------------------------
# Token shift with per-sequence state, query/key norm followed by rotation,
# chunk-masked differential attention, the HGRN2 recurrence, sigmoid routing
# and gated experts whose input carries the routing weight.
# ---------------------------------------------------------------------------


def token_shift_state(x: torch.Tensor, weight: torch.Tensor, state: torch.Tensor,
                      seq_start_loc, seq_lens, state_slots,
                      out_dtype: torch.dtype) -> torch.Tensor:
    """out_t = x_t + (x_(t-1) - x_t) * weight per sequence, x [T, W] f32; the
    row before a portion's first row comes from ``state[slot]`` (f32 [slots,
    W]), the row before position 0 is zero; ``state[slot]`` then becomes the
    portion's last row."""
    out = torch.zeros(x.shape, dtype=out_dtype, device=x.device)
    wf = weight.float()
    for a, b, start, slot in _seq_iter(seq_start_loc, seq_lens, state_slots):
        if slot < 0:
            continue
        xs = x[a:b].float()
        first = state[slot].float() if start > 0 else torch.zeros_like(xs[0])
        prev = torch.cat([first.unsqueeze(0), xs[:-1]], dim=0)
        out[a:b] = (xs + (prev - xs) * wf).to(out_dtype)
        state[slot] = xs[-1]
    return out


def qk_norm_rope_cache_write(q, k, v, q_weight, k_weight, eps, positions, inv_freq,
                             rot_dims: int, k_cache, v_cache, slot_mapping):
    """Per-head RMS norm of q [T, H, dim] and k [T, G, dim] (plain weight),
    then rotation of the first ``rot_dims`` dims (dim i with i + rot_dims/2,
    f32 angles position * inv_freq[i]); rotated keys and v [T, Gv, vdim] go to
    the paged cache.  Returns the queries, contiguous."""
    def norm_rot(x, w):
        xf = x.float()
        xf = xf * torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + eps) * w.float()
        if rot_dims:
            xf = xf.contiguous()
            rope_partial(xf, positions, inv_freq, 0, rot_dims)
        return xf
    qf, kf = norm_rot(q, q_weight), norm_rot(k, k_weight)
    ok = slot_mapping >= 0
    sm = slot_mapping[ok]
    bs = k_cache.shape[1]
    blk = torch.div(sm, bs, rounding_mode="floor")
    k_cache[blk, sm % bs] = kf[ok].to(k_cache.dtype)
    v_cache[blk, sm % bs] = v[ok].to(v_cache.dtype)
    return qf.to(q.dtype).contiguous()


def chunk_attention(q, k_cache, v_cache, block_tables, query_start_loc, seq_lens,
                    scale: float, chunk: int) -> torch.Tensor:
    """Causal grouped-query softmax attention of each sequence's tail rows over
    the paged cache in which position i sees j <= i only when floor(i / chunk)
    = floor(j / chunk) (chunk 0: every j <= i).  q [T, H, dim]; key head of
    query head h is h // (H / G); the value cache may hold fewer heads Gv than
    the key cache: key head g reads value head g % Gv.  Returns f32 [T, H,
    vdim]."""
    nh, ng, gv = q.shape[1], k_cache.shape[2], v_cache.shape[2]
    group = nh // ng
    out = torch.zeros((q.shape[0], nh, v_cache.shape[-1]), dtype=torch.float32,
                      device=q.device)
    qs = query_start_loc.tolist()
    lens = seq_lens.tolist()
    for i in range(len(lens)):
        s, e = qs[i], qs[i + 1]
        n, ctx = e - s, lens[i]
        if n == 0 or ctx == 0:
            continue
        k, v = _gather_kv(k_cache, v_cache, block_tables[i], ctx)
        kf = k.float().repeat_interleave(group, dim=1)
        vh = torch.arange(nh, device=q.device) // group % gv
        vf = v.float()[:, vh]
        scores = torch.einsum("qhd,shd->hqs", q[s:e].float(), kf) * scale
        kpos = torch.arange(ctx, device=q.device)
        qpos = torch.arange(ctx - n, ctx, device=q.device)
        mask = kpos[None, :] > qpos[:, None]
        if chunk > 0:
            mask = mask | (torch.div(qpos[:, None], chunk, rounding_mode="floor")
                           != torch.div(kpos[None, :], chunk, rounding_mode="floor"))
        scores.masked_fill_(mask.unsqueeze(0), float("-inf"))
        out[s:e] = torch.einsum("hqs,shd->qhd", torch.softmax(scores, dim=-1), vf)
    return out


def diff_combine(a: torch.Tensor, lam: float, out_scale: float, eps: float,
                 gate: torch.Tensor | None, out_dtype: torch.dtype) -> torch.Tensor:
    """a [T, 2, H, vdim] f32, the two maps' outputs: o = a[:, 0] - lam * a[:, 1],
    divided by its root mean square over vdim (eps inside the root), times
    ``out_scale``, times sigmoid(gate[t, h]) when a gate [T, H] is given.
    Returns [T, H * vdim]."""
    o = a[:, 0].float() - lam * a[:, 1].float()
    o = o * torch.rsqrt(o.pow(2).mean(dim=-1, keepdim=True) + eps) * out_scale
    if gate is not None:
        o = o * torch.sigmoid(gate.float()).unsqueeze(-1)
    return o.to(out_dtype).reshape(o.shape[0], -1)


def hgrn2_scan(q: torch.Tensor, f: torch.Tensor, v: torch.Tensor, f_bias: torch.Tensor,
               lower: torch.Tensor, state: torch.Tensor, seq_start_loc, seq_lens,
               state_slots) -> torch.Tensor:
    """Gated linear recurrence whose forget gate also sets what is written.
    q, f [T, H, dim] (projections, before their activations), v [T, H, vdim];
    g = lower + (1 - lower) * sigmoid(f + f_bias) per channel; per head
    S_t = diag(g_t) S_(t-1) + (1 - g_t) v_t^T, o_t = S_t^T silu(q_t).  State
    [slots, H, vdim, dim] f32, advanced in place; a sequence that starts in
    this step starts from zero.  Returns o [T, H * vdim] f32."""
    t, nh, d = q.shape
    dv = v.shape[-1]
    qf = q.float()
    qf = qf * torch.sigmoid(qf)
    lo = lower.float().view(nh, d)
    g = lo + (1.0 - lo) * torch.sigmoid(f.float() + f_bias.float().view(nh, d))
    vf = v.float()
    out = torch.zeros((t, nh, dv), dtype=torch.float32, device=q.device)
    for a, b, start, slot in _seq_iter(seq_start_loc, seq_lens, state_slots):
        if slot < 0:
            continue
        s = state[slot].clone() if start > 0 else torch.zeros_like(state[slot])
        for i in range(a, b):
            s = g[i].unsqueeze(1) * s + vf[i].unsqueeze(2) * (1.0 - g[i]).unsqueeze(1)
            out[i] = torch.einsum("hvd,hd->hv", s, qf[i])
        state[slot] = s
    return out.view(t, nh * dv)


def group_rms_norm(y: torch.Tensor, weight: torch.Tensor, groups: int, eps: float,
                   out_dtype: torch.dtype) -> torch.Tensor:
    """RMS norm of y [T, C] in ``groups`` equal parts, times weight [C]."""
    t, c = y.shape
    yg = y.float().view(t, groups, c // groups)
    yg = yg * torch.rsqrt(yg.pow(2).mean(dim=-1, keepdim=True) + eps)
    return (yg.reshape(t, c) * weight.float()).to(out_dtype)


def moe_route_sigmoid(logits: torch.Tensor, top: int):
    """s = sigmoid(logits) [T, E] f32; the ``top`` largest are chosen (ties:
    the lower index); weights = their s as they are.  Returns (dense [T, E]
    f32: weight or 0, ids [T, top] int32, weights [T, top] f32)."""
    s = torch.sigmoid(logits.float())
    order = torch.sort(s, dim=-1, descending=True, stable=True).indices[:, :top]
    w = torch.gather(s, 1, order)
    return torch.zeros_like(s).scatter_(1, order, w), order.to(torch.int32), w


def silu_mul_scaled(gu: torch.Tensor, col_scale: torch.Tensor) -> torch.Tensor:
    """gu [T, E, 2, ff] flattened (expert-major, gate rows then up rows);
    out[t, e, j] = silu(w * gate) * (w * up) with w = col_scale[t, e]: the
    gated activation of an expert whose input was multiplied by w."""
    t, e = col_scale.shape
    z = gu.float().view(t, e, 2, -1) * col_scale.float().view(t, e, 1, 1)
    g, u = z[:, :, 0], z[:, :, 1]
    return (g * torch.sigmoid(g) * u).to(gu.dtype).reshape(t, -1)
