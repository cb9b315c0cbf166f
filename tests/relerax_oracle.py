"""A plain, slow implementation of the Relerax design, one function per
mechanism, written from the design's equations in float64.  It shares no code
with the package: tests compare the engine against it.

Notation: x is the residual stream [n, width] of ONE sequence, processed whole;
position t is row t.  Attention is computed key by key in the expanded form
(per-head keys and values are materialised from the latent), not in the folded
form the kernels use.
"""

from __future__ import annotations

import json
import math
import os

import torch

F64 = torch.float64


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def rms_norm(x, w, eps):
    return unit_rms(x, eps) * w


def relu_squared(z):
    return torch.clamp(z, min=0.0) ** 2


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


# -- rotation ---------------------------------------------------------------

def scaled_frequencies(rot: dict) -> tuple[list[float], float]:
    """Frequencies f_i of the pairs (2i, 2i+1) and the factor that multiplies
    cos and sin.  Without rot["scaling"]: f_i = base^(-2i/dims), factor 1.
    With it (factor s, original length L, fast, slow): pairs that turn often
    keep f_i, pairs that turn rarely get f_i / s, a linear ramp over the pair
    index in between; cos and sin are multiplied by 0.1 ln(s) + 1."""
    base, dims = float(rot["base"]), int(rot["dims"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    s, orig = float(sc["factor"]), float(sc["original"])

    def pair_index_of(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(pair_index_of(float(sc["fast"]))), 0)
    hi = min(math.ceil(pair_index_of(float(sc["slow"]))), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / s * ramp + fi * (1.0 - ramp))
    return out, 0.1 * math.log(s) + 1.0


def rotate_pairs(v, pos, freqs, mag):
    """v [..., d], d >= 2 len(freqs): neighbouring dims (2i, 2i+1) of the first
    2 len(freqs) dims are rotated by pos * freqs[i]; the rest pass."""
    out = v.clone()
    for i, f in enumerate(freqs):
        a = pos * f
        c, s = math.cos(a) * mag, math.sin(a) * mag
        u, w = v[..., 2 * i], v[..., 2 * i + 1]
        out[..., 2 * i] = u * c - w * s
        out[..., 2 * i + 1] = w * c + u * s
    return out


# -- mixers -----------------------------------------------------------------

def windowed_sink_attention(h, w_q, w_k, w_g, w_o, *, heads, kv_heads, dim, scale,
                            window, rot):
    """Grouped-query attention whose values are the unrotated keys, with a
    sliding window, a denominator that holds one extra 1 (a sink of score 0
    with no value) and an elementwise sigmoid output gate."""
    n = h.shape[0]
    freqs, mag = scaled_frequencies(rot)
    q = (h @ w_q.T).view(n, heads, dim)
    k = (h @ w_k.T).view(n, kv_heads, dim)
    v = k.clone()
    qr = torch.stack([rotate_pairs(q[t], t, freqs, mag) for t in range(n)])
    kr = torch.stack([rotate_pairs(k[t], t, freqs, mag) for t in range(n)])
    per = heads // kv_heads
    out = torch.zeros(n, heads * dim, dtype=h.dtype)
    for hh in range(heads):
        g = hh // per
        for i in range(n):
            lo = max(0, i - window + 1) if window else 0
            s = torch.stack([(qr[i, hh] @ kr[j, g]) * scale for j in range(lo, i + 1)])
            m = max(float(s.max()), 0.0)
            e = torch.exp(s - m)
            p = e / (e.sum() + math.exp(-m))
            out[i, hh * dim:(hh + 1) * dim] = p @ v[lo:i + 1, g]
    out = out * sigmoid(h @ w_g.T)
    return out @ w_o.T


def latent_attention(h, w_q, w_dkv, w_norm, w_uk, w_uv, w_g, w_o, *, heads, dim,
                     rot_dim, vdim, rank, scale, eps, rot):
    """Causal attention whose keys and values are up-projections of one normed
    latent per token, plus one rotated key part shared by all heads; ordinary
    softmax; one sigmoid gate per head."""
    n = h.shape[0]
    freqs, mag = scaled_frequencies(rot)
    q = (h @ w_q.T).view(n, heads, dim + rot_dim)
    dkv = h @ w_dkv.T
    c = rms_norm(dkv[:, :rank], w_norm, eps)
    kr = torch.stack([rotate_pairs(dkv[t, rank:], t, freqs, mag) for t in range(n)])
    gate = sigmoid(h @ w_g.T)                                  # [n, heads]
    out = torch.zeros(n, heads * vdim, dtype=h.dtype)
    for hh in range(heads):
        k_h = c @ w_uk[hh * dim:(hh + 1) * dim].T
        v_h = c @ w_uv[hh * vdim:(hh + 1) * vdim].T
        for i in range(n):
            q_rot = rotate_pairs(q[i, hh, dim:], i, freqs, mag)
            s = torch.stack([(q[i, hh, :dim] @ k_h[j] + q_rot @ kr[j]) * scale
                             for j in range(i + 1)])
            p = torch.softmax(s, dim=0)
            out[i, hh * vdim:(hh + 1) * vdim] = (p @ v_h[:i + 1]) * gate[i, hh]
    return out @ w_o.T


# -- feed-forward -----------------------------------------------------------

def dense_ff(h, w_up, b_up, w_down, b_down):
    return relu_squared(h @ w_up.T + b_up) @ w_down.T + b_down


def routed_ff(h, w_router, correction, experts, *, top, identity, margins=None):
    """experts: list of (w_up, w_down); the last ``identity`` router outputs
    are experts that return their input.  ``margins`` (a list) receives, per
    token, the gap between the last chosen and the first unchosen choice
    score: a small gap is a close call that rounding may decide otherwise."""
    n = h.shape[0]
    z = h @ w_router.T
    s = torch.softmax(z, dim=-1)
    choice = s + correction
    out = torch.zeros_like(h)
    real = len(experts)
    for t in range(n):
        ranked = sorted(range(real + identity), key=lambda e: (-float(choice[t, e]), e))
        order = ranked[:top]
        if margins is not None:
            margins.append(float(choice[t, ranked[top - 1]] - choice[t, ranked[top]])
                           if top < real + identity else float("inf"))
        tot = sum(float(s[t, e]) for e in order) + 1e-20
        for e in order:
            wgt = float(s[t, e]) / tot
            if e >= real:
                out[t] += wgt * h[t]
            else:
                up, down = experts[e]
                out[t] += wgt * (relu_squared(h[t] @ up.T) @ down.T)
    return out


# -- the model --------------------------------------------------------------

def forward(cfg: dict, w: dict, tokens: list[int], layers_out: list | None = None,
            margins_out: list | None = None):
    """Logits [n, vocab] of one whole sequence.  ``margins_out`` receives one
    list per routed layer with every token's router margin (see routed_ff)."""
    w = {k: v.to(F64) for k, v in w.items()}
    eps = float(cfg["norm"]["eps"])
    x = w["embed"][torch.tensor(tokens)]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        m = layer["mixer"]
        h1 = rms_norm(x, w[p + "norm1"], eps)
        if layer["type"] == "attention":
            assert int(m.get("vdim", m["dim"])) == int(m["dim"])
            y = windowed_sink_attention(
                h1, w[p + "mix.q"], w[p + "mix.k"], w[p + "mix.g"], w[p + "mix.o"],
                heads=m["heads"], kv_heads=m["kv_heads"], dim=m["dim"], scale=m["scale"],
                window=int((m.get("mask") or {}).get("size") or 0), rot=m["rot"])
        elif layer["type"] == "latent_attention":
            rot = dict(m["rot"])
            rot["dims"] = m["rot_dim"]
            y = latent_attention(
                h1, w[p + "mix.q"], w[p + "mix.dkv"], w[p + "mix.dkv.norm"],
                w[p + "mix.uk"], w[p + "mix.uv"], w[p + "mix.g"], w[p + "mix.o"],
                heads=m["heads"], dim=m["dim"], rot_dim=m["rot_dim"], vdim=m["vdim"],
                rank=m["kv_rank"], scale=m["scale"], eps=eps, rot=rot)
        else:
            raise ValueError(layer["type"])
        mlp = layer.get("mlp")
        if mlp is not None:
            h2 = rms_norm(x, w[p + "norm2"], eps)
            if mlp["kind"] == "dense":
                y = y + dense_ff(h2, w[p + "mlp.up"], w[p + "mlp.up.b"],
                                 w[p + "mlp.down"], w[p + "mlp.down.b"])
            else:
                r = mlp["router"]
                experts = [(w[f"{p}mlp.e{e}.up"], w[f"{p}mlp.e{e}.down"])
                           for e in range(int(r["experts"]))]
                m_list = [] if margins_out is not None else None
                y = y + routed_ff(h2, w[p + "mlp.router"], w[p + "mlp.correction"], experts,
                                  top=int(r["top"]), identity=int(r.get("identity", 0)),
                                  margins=m_list)
                if margins_out is not None:
                    margins_out.append(m_list)
        x = x + y
        if layers_out is not None:
            layers_out.append(x.clone())
    return rms_norm(x, w["final.norm"], eps) @ w["head"].T


# -- making small models ----------------------------------------------------

def tensor_shapes(cfg: dict) -> dict:
    width, vocab = cfg["width"], cfg["vocab"]
    shapes = {"embed": (vocab, width), "final.norm": (width,), "head": (vocab, width)}
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        m = layer["mixer"]
        shapes[p + "norm1"] = (width,)
        if layer["type"] == "attention":
            shapes[p + "mix.q"] = (m["heads"] * m["dim"], width)
            shapes[p + "mix.k"] = (m["kv_heads"] * m["dim"], width)
            shapes[p + "mix.g"] = (m["heads"] * m["dim"], width)
            shapes[p + "mix.o"] = (width, m["heads"] * m["dim"])
        else:
            shapes[p + "mix.q"] = (m["heads"] * (m["dim"] + m["rot_dim"]), width)
            shapes[p + "mix.dkv"] = (m["kv_rank"] + m["rot_dim"], width)
            shapes[p + "mix.dkv.norm"] = (m["kv_rank"],)
            shapes[p + "mix.uk"] = (m["heads"] * m["dim"], m["kv_rank"])
            shapes[p + "mix.uv"] = (m["heads"] * m["vdim"], m["kv_rank"])
            shapes[p + "mix.g"] = (m["heads"], width)
            shapes[p + "mix.o"] = (width, m["heads"] * m["vdim"])
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        shapes[p + "norm2"] = (width,)
        if mlp["kind"] == "dense":
            shapes[p + "mlp.up"] = (mlp["ff"], width)
            shapes[p + "mlp.up.b"] = (mlp["ff"],)
            shapes[p + "mlp.down"] = (width, mlp["ff"])
            shapes[p + "mlp.down.b"] = (width,)
        else:
            r = mlp["router"]
            ff = mlp["expert"]["ff"]
            for e in range(r["experts"]):
                shapes[f"{p}mlp.e{e}.up"] = (ff, width)
                shapes[f"{p}mlp.e{e}.down"] = (width, ff)
            shapes[p + "mlp.router"] = (r["experts"] + r.get("identity", 0), width)
            shapes[p + "mlp.correction"] = (r["experts"] + r.get("identity", 0),)
    return shapes


def random_weights(cfg: dict, seed: int = 0, dtype=torch.bfloat16) -> dict:
    """Weights with O(1) activations everywhere, rounded to ``dtype`` so that
    engine and oracle start from the same numbers."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".")[-1]
        if "norm" in leaf:
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        elif leaf == "b":
            t = 0.3 * torch.randn(shape, generator=g)
        elif leaf == "correction":
            t = 0.1 * torch.randn(shape, generator=g)
        elif leaf == "router":
            t = 2.0 * torch.randn(shape, generator=g) / math.sqrt(shape[-1])
        else:
            t = torch.randn(shape, generator=g) / math.sqrt(shape[-1])
        out[name] = t.to(dtype)
    return out


def write_model(path: str, cfg: dict, weights: dict) -> None:
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in weights.items()},
              os.path.join(path, "model.safetensors"))
