"""A plain, slow implementation of the Gumozen design, one function per
mechanism, written from the design's equations in float64.  It shares no code
with the package: tests compare the engine against it.

Notation: x is the residual stream [n, width] of ONE sequence, processed whole;
position t is row t.  Attention is computed query by query over explicit key
lists, the recurrence token by token, the experts token by token.
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


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def silu(z):
    return z * sigmoid(z)


# -- token shift --------------------------------------------------------------

def token_shift(x, w):
    """Row t becomes x_t + (x_(t-1) - x_t) * w, with the rows as they were
    before any blending and a zero row before the first."""
    out = torch.empty_like(x)
    for t in range(x.shape[0]):
        prev = x[t - 1] if t > 0 else torch.zeros_like(x[0])
        out[t] = x[t] + (prev - x[t]) * w
    return out


# -- rotation -----------------------------------------------------------------

def stepped_frequencies(rot: dict) -> list[float]:
    """f_i = base^(-2i/dims) for the dims/2 pairs (i, i + dims/2).  With
    rot["scaling"] = {factor, low, high, original}: a pair whose wavelength
    2 pi / f is shorter than original/high keeps f, one longer than
    original/low gets f / factor, and in between the two are blended with
    s = (original / wavelength - low) / (high - low): (1 - s) f / factor + s f."""
    base, dims = float(rot["base"]), int(rot["dims"])
    out = []
    sc = rot.get("scaling")
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if sc:
            wave = 2.0 * math.pi / f
            short, long_ = sc["original"] / sc["high"], sc["original"] / sc["low"]
            if wave > long_:
                f = f / sc["factor"]
            elif wave >= short:
                s = (sc["original"] / wave - sc["low"]) / (sc["high"] - sc["low"])
                f = (1.0 - s) * f / sc["factor"] + s * f
        out.append(f)
    return out


def rotate_half_split(v, pos: int, freqs: list[float]):
    """v [dim]: dims i and i + len(freqs) turn by pos * f_i, the rest stay."""
    out = v.clone()
    half = len(freqs)
    for i, f in enumerate(freqs):
        a = pos * f
        c, s = math.cos(a), math.sin(a)
        out[i] = v[i] * c - v[i + half] * s
        out[i + half] = v[i + half] * c + v[i] * s
    return out


# -- mixers -------------------------------------------------------------------

def differential_attention(h, w, *, heads, kv_heads, dim, vdim, scale, diff, chunk, rot,
                           eps):
    """w: q [heads*2*dim, W] (head by head: map 1, map 2), k [kv_heads*2*dim, W],
    v [kv_heads*vdim, W], q.norm, k.norm [dim], lq1, lk1, lq2, lk2 [dim],
    g [heads, W], o [W, heads*vdim]."""
    n = h.shape[0]
    q = (h @ w["q"].T).view(n, heads, 2, dim)
    k = (h @ w["k"].T).view(n, kv_heads, 2, dim)
    v = (h @ w["v"].T).view(n, kv_heads, vdim)
    gate = sigmoid(h @ w["g"].T)                              # [n, heads]
    q = rms_norm(q, w["q.norm"], eps)
    k = rms_norm(k, w["k.norm"], eps)
    freqs = stepped_frequencies(rot) if rot and rot.get("dims") else []
    for t in range(n):
        for m in range(2):
            for a in range(heads):
                q[t, a, m] = rotate_half_split(q[t, a, m], t, freqs)
            for b in range(kv_heads):
                k[t, b, m] = rotate_half_split(k[t, b, m], t, freqs)
    lam = (math.exp(float((w["lq1"] * w["lk1"]).sum()))
           - math.exp(float((w["lq2"] * w["lk2"]).sum())) + diff)
    per = heads // kv_heads
    out = torch.zeros(n, heads, vdim, dtype=F64)
    for t in range(n):
        first = (t // chunk) * chunk if chunk else 0
        keys = list(range(first, t + 1))
        for a in range(heads):
            b = a // per
            maps = []
            for m in range(2):
                s = torch.stack([(q[t, a, m] * k[j, b, m]).sum() * scale for j in keys])
                p = torch.exp(s - s.max())
                p = p / p.sum()
                maps.append(sum(p[i] * v[j, b] for i, j in enumerate(keys)))
            o = maps[0] - lam * maps[1]
            out[t, a] = unit_rms(o, eps) * (1.0 - diff) * gate[t, a]
    return out.reshape(n, heads * vdim) @ w["o"].T


def hgrn2(h, w, *, heads, dim, vdim, eps):
    """w: q, f [heads*dim, W], f.b, lower [heads*dim], v [heads*vdim, W],
    norm [vdim], o [W, heads*vdim]."""
    n = h.shape[0]
    q = silu(h @ w["q"].T).view(n, heads, dim)
    v = (h @ w["v"].T).view(n, heads, vdim)
    lo = w["lower"]
    f = (lo + (1.0 - lo) * sigmoid(h @ w["f"].T + w["f.b"])).view(n, heads, dim)
    state = torch.zeros(heads, dim, vdim, dtype=F64)
    out = torch.zeros(n, heads, vdim, dtype=F64)
    for t in range(n):
        for a in range(heads):
            state[a] = f[t, a].unsqueeze(1) * state[a] \
                + (1.0 - f[t, a]).unsqueeze(1) * v[t, a].unsqueeze(0)
            out[t, a] = state[a].T @ q[t, a]
    out = rms_norm(out, w["norm"], eps)
    return out.reshape(n, heads * vdim) @ w["o"].T


def latent_attention(h, w, latent_in, *, heads, dim, vdim, scale, eps):
    """w: dq [q_rank, W], dq.norm, uq [heads*dim, q_rank], uk [heads*dim, rank],
    uv [heads*vdim, rank], o, and with a latent of its own dkv [rank, W],
    dkv.norm.  ``latent_in``: another layer's latent rows [n, rank], or None.
    Returns (output, the latent rows it used)."""
    n = h.shape[0]
    q = (rms_norm(h @ w["dq"].T, w["dq.norm"], eps) @ w["uq"].T).view(n, heads, dim)
    c = latent_in if latent_in is not None else rms_norm(h @ w["dkv"].T, w["dkv.norm"], eps)
    k = (c @ w["uk"].T).view(n, heads, dim)
    v = (c @ w["uv"].T).view(n, heads, vdim)
    out = torch.zeros(n, heads, vdim, dtype=F64)
    for t in range(n):
        for a in range(heads):
            s = torch.stack([(q[t, a] * k[j, a]).sum() * scale for j in range(t + 1)])
            p = torch.exp(s - s.max())
            p = p / p.sum()
            out[t, a] = sum(p[j] * v[j, a] for j in range(t + 1))
    return out.reshape(n, heads * vdim) @ w["o"].T, c


# -- feed-forward ---------------------------------------------------------------

def routed_gated_ff(h, w_router, experts, *, top, margins=None):
    """experts: list of (gate [ff, W], up [ff, W], down [W, ff]).  Scores are
    sigmoid(router h); the ``top`` largest choose the experts and weigh them as
    they are; the weight multiplies the expert's input.  ``margins`` collects
    per token the gap between the last chosen and the first unchosen score."""
    n = h.shape[0]
    out = torch.zeros_like(h)
    for t in range(n):
        s = sigmoid(w_router @ h[t])
        order = sorted(range(len(experts)), key=lambda e: (-float(s[e]), e))
        if margins is not None:
            margins.append(float(s[order[top - 1]] - s[order[top]])
                           if top < len(experts) else 1.0)
        for e in order[:top]:
            gate, up, down = experts[e]
            x = s[e] * h[t]
            out[t] += down @ (silu(gate @ x) * (up @ x))
    return out


# -- the model ----------------------------------------------------------------

def _sub(w: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v.to(F64) for k, v in w.items() if k.startswith(prefix)}


def forward(cfg: dict, w: dict, tokens: list[int], layers_out: list | None = None,
            margins_out: list | None = None):
    """Logits [n, vocab] of one sequence; ``layers_out`` collects the stream
    after every layer, ``margins_out`` each routed layer's per-token margins."""
    eps = cfg["norm"]["eps"]
    x = rms_norm(w["embed"].to(F64)[torch.tensor(tokens)], w["embed.norm"].to(F64), eps)
    latents = {}
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        m = layer["mixer"]
        t = _sub(w, p + "mix.")
        h = token_shift(x, w[p + "shift"].to(F64))
        if layer["type"] == "attention":
            y = differential_attention(
                h, t, heads=m["heads"], kv_heads=m["kv_heads"], dim=m["dim"], vdim=m["vdim"],
                scale=m["scale"], diff=m["diff"], chunk=(m.get("mask") or {}).get("size", 0),
                rot=m.get("rot"), eps=eps)
        elif layer["type"] == "hgrn2":
            y = hgrn2(h, t, heads=m["heads"], dim=m["dim"], vdim=m["vdim"], eps=eps)
        else:
            src = m.get("kv_from")
            y, latents[i] = latent_attention(
                h, t, None if src is None else latents[src], heads=m["heads"], dim=m["dim"],
                vdim=m["vdim"], scale=m["scale"], eps=eps)
        x = x + rms_norm(y, w[p + "norm1"].to(F64), eps) * w[p + "ls1"].to(F64)
        mlp = layer.get("mlp")
        if mlp is not None:
            ne = mlp["router"]["experts"]
            ex = [tuple(w[f"{p}mlp.e{e}.{n}"].to(F64) for n in ("gate", "up", "down"))
                  for e in range(ne)]
            margins = [] if margins_out is not None else None
            y = routed_gated_ff(x, w[p + "mlp.router"].to(F64), ex, top=mlp["router"]["top"],
                                margins=margins)
            if margins_out is not None:
                margins_out.append(margins)
            x = x + rms_norm(y, w[p + "norm2"].to(F64), eps) * w[p + "ls2"].to(F64)
        if layers_out is not None:
            layers_out.append(x.clone())
    return rms_norm(x, w["final.norm"].to(F64), eps) @ w["head"].to(F64).T


# -- making small models --------------------------------------------------------

def tensor_shapes(cfg: dict) -> dict:
    width, vocab = cfg["width"], cfg["vocab"]
    shapes = {"embed": (vocab, width), "embed.norm": (width,), "final.norm": (width,),
              "head": (vocab, width)}
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        m = layer["mixer"]
        for n in ("norm1", "ls1", "shift"):
            shapes[p + n] = (width,)
        x = p + "mix."
        if layer["type"] == "attention":
            nh, ng, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            shapes.update({x + "q": (nh * 2 * d, width), x + "k": (ng * 2 * d, width),
                           x + "v": (ng * dv, width), x + "g": (nh, width),
                           x + "o": (width, nh * dv), x + "q.norm": (d,), x + "k.norm": (d,)})
            for n in ("lq1", "lk1", "lq2", "lk2"):
                shapes[x + n] = (d,)
        elif layer["type"] == "hgrn2":
            nh, d, dv = m["heads"], m["dim"], m["vdim"]
            shapes.update({x + "q": (nh * d, width), x + "f": (nh * d, width),
                           x + "f.b": (nh * d,), x + "lower": (nh * d,),
                           x + "v": (nh * dv, width), x + "norm": (dv,),
                           x + "o": (width, nh * dv)})
        else:
            nh, d, dv, rank, qr = m["heads"], m["dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            shapes.update({x + "dq": (qr, width), x + "dq.norm": (qr,), x + "uq": (nh * d, qr),
                           x + "uk": (nh * d, rank), x + "uv": (nh * dv, rank),
                           x + "o": (width, nh * dv)})
            if m.get("kv_from") is None:
                shapes.update({x + "dkv": (rank, width), x + "dkv.norm": (rank,)})
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        shapes[p + "norm2"] = (width,)
        shapes[p + "ls2"] = (width,)
        ff = mlp["expert"]["ff"]
        for e in range(mlp["router"]["experts"]):
            shapes[f"{p}mlp.e{e}.gate"] = (ff, width)
            shapes[f"{p}mlp.e{e}.up"] = (ff, width)
            shapes[f"{p}mlp.e{e}.down"] = (width, ff)
        shapes[p + "mlp.router"] = (mlp["router"]["experts"], width)
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
        elif leaf in ("ls1", "ls2"):
            t = 0.5 + 0.2 * torch.randn(shape, generator=g)
        elif leaf == "shift":
            t = torch.rand(shape, generator=g)
        elif leaf == "lower":
            t = 0.9 * torch.rand(shape, generator=g)
        elif leaf == "b":
            t = 0.5 * torch.randn(shape, generator=g)
        elif leaf in ("lq1", "lk1", "lq2", "lk2"):
            t = 0.3 * torch.randn(shape, generator=g)
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
