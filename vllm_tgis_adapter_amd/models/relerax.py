"""Relerax: a decoder-only model with an f32 residual stream whose layers are
parallel blocks with two norms,

    x <- x + mixer(norm1(x)) + ff(norm2(x)),

both RMS norms (plain weight) of the same x, so they share one statistic.  The
mixer of a layer is one of

  attention         grouped-query softmax attention; rot.dims leading dims of
                    every head are rotated (neighbouring dims form a pair,
                    frequencies stretched the YaRN way); there is no value
                    projection, the unrotated key projections serve as values;
                    keys further back than mask.size - 1 positions are masked;
                    the softmax denominator is 1 + sum(exp(s)), i.e. a sink
                    with logit 0 and no value; W_o reads the heads multiplied
                    elementwise by sigmoid(W_g h)
  latent_attention  causal attention over one cached latent row per token
                    (RMS-normed latent + one rotated key part shared by all
                    heads), ordinary softmax, head h's output times
                    sigmoid(W_g h)_h

and the feed-forward is dense (squared relu, biases), a mixture of small
squared-relu experts plus identity experts (output = input) behind a softmax
router (top-k picked on score + correction, weighted by the renormalised plain
scores), or absent.  The head is the final RMS norm and a linear map.

Sizes and constants all come from config.json:

  vocab, width, norm.eps, layers[i] = {type, mixer{...}, mlp{kind, ...} | null}
  attention mixer:   heads, kv_heads, dim, vdim, scale, mask.size, rot{base,
                     dims, scaling{factor, original, fast, slow}}
  latent mixer:      heads, dim, rot_dim, vdim, kv_rank, scale, rot{base,
                     scaling{...}}
  mlp dense:         ff          mlp moe: expert.ff, router{experts, identity, top}

Tensors: embed, final.norm, head, l<i>.{norm1, norm2}, l<i>.mix.{q, k, g, o} or
l<i>.mix.{q, dkv, dkv.norm, uk, uv, g, o}, l<i>.mlp.{up, up.b, down, down.b} or
l<i>.mlp.{router, correction, e<j>.up, e<j>.down}.
"""

from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from .. import ops
from ..engine.config import ModelConfig
from ..engine.metadata import AttnMetadata
from ..parallel import get_tp_world_size
from .blocks import (
    BiasedDenseMLP,
    LatentAttention,
    RotatedAttention,
    RoutedExperts,
    _f32_param,
)

# positions are unbounded in this design (rotary only); the default bounds
# block tables and capture buffers and can be raised with --max-model-len
_DEFAULT_MAX_LEN = 32768

# the softmax of the attention mixer has a sink with this logit: exp(0) = 1
# joins the denominator
ATTENTION_SINK_LOGIT = 0.0


def build_mixer(kind: str, m: dict, width: int, eps: float, dtype: torch.dtype):
    rot = m.get("rot") or {}
    if kind == "attention":
        dim = int(m["dim"])
        return RotatedAttention(
            width, heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])),
            dim=dim, vdim=int(m.get("vdim", dim)), scale=float(m["scale"]),
            window=int((m.get("mask") or {}).get("size") or 0),
            sink=ATTENTION_SINK_LOGIT, rot_base=float(rot.get("base", 10000.0)),
            rot_dims=int(rot.get("dims", 0)), rot_interleaved=True,
            rot_scaling=rot.get("scaling"), values_from_keys=True, gate="elementwise",
            dtype=dtype)
    if kind == "latent_attention":
        rot_dim = int(m["rot_dim"])
        return LatentAttention(
            width, heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=rot_dim,
            vdim=int(m["vdim"]), rank=int(m["kv_rank"]), scale=float(m["scale"]),
            window=0, rot_base=float(rot.get("base", 10000.0)), rot_dims=rot_dim,
            eps=eps, kv_owner=True, has_sink=False, dtype=dtype, rot_interleaved=True,
            rot_scaling=rot.get("scaling"), head_gate=True, two_term_weights=True)
    raise ValueError(f"unknown mixer type {kind!r}")


def build_ff(mlp: Optional[dict], width: int, dtype: torch.dtype):
    if mlp is None:
        return None
    kind = mlp.get("kind", "dense")
    if kind == "dense":
        return BiasedDenseMLP(width, int(mlp["ff"]), dtype)
    if kind == "moe":
        r = mlp["router"]
        return RoutedExperts(width, experts=int(r["experts"]), identity=int(r.get("identity", 0)),
                             top=int(r["top"]), ff=int(mlp["expert"]["ff"]), dtype=dtype)
    raise ValueError(f"unknown feed-forward kind {kind!r}")


def model_config_from_json(model: str, hf: dict) -> ModelConfig:
    layers = hf["layers"]
    for i, e in enumerate(layers):
        if e.get("type") not in ("attention", "latent_attention"):
            raise ValueError(f"layer {i}: unknown mixer type {e.get('type')!r}")
    att = [e["mixer"] for e in layers if e["type"] == "attention"]
    moe = [e["mlp"] for e in layers if (e.get("mlp") or {}).get("kind") == "moe"]
    ffs = [int(e["mlp"]["ff"]) for e in layers if (e.get("mlp") or {}).get("kind", "dense") == "dense"
           and e.get("mlp")] + [int(m["expert"]["ff"]) for m in moe]
    return ModelConfig(
        model=model,
        architecture="relerax",
        vocab_size=int(hf["vocab"]),
        hidden_size=int(hf["width"]),
        intermediate_size=max(ffs, default=0),
        num_layers=len(layers),
        num_heads=max(int(e["mixer"]["heads"]) for e in layers),
        num_kv_heads=max((int(a.get("kv_heads", a["heads"])) for a in att), default=1),
        head_dim=max((int(a["dim"]) for a in att), default=1),
        rope_theta=0.0,
        rms_norm_eps=float((hf.get("norm") or {}).get("eps", 1e-5)),
        max_model_len=int(hf.get("max_len", _DEFAULT_MAX_LEN)),
        tie_word_embeddings=False,
        dtype=torch.bfloat16,
        # num_experts stays 0: that field describes the mixtral expert layout
        # (and gates its capture rules); the routed layers here are shape-static
        hf_config=hf,
    )


def native_extensions(cfg: ModelConfig) -> list[str]:
    """Stream ops, rotation + cache write, any-shape attention, gates and
    router live in the sequence extension; latent attention has its own; the
    MFMA attention kernels (alone, without the rest of their extension) are
    needed when an attention mixer has a shape they take."""
    need = ["_C_seq"]
    layers = cfg.hf_config["layers"]
    if any(e.get("type") == "latent_attention" for e in layers):
        need.append("_C_lat")
    for e in layers:
        if e.get("type") != "attention":
            continue
        a = e["mixer"]
        dim = int(a["dim"])
        if ops.windowed_attention_uses_matrix_cores(
                cfg.dtype, int(a["heads"]), int(a.get("kv_heads", a["heads"])), dim,
                int(a.get("vdim", dim))):
            need.append("_C_attn")
            break
    return need


class ReleraxLayer(nn.Module):
    def __init__(self, idx: int, entry: dict, width: int, eps: float, dtype: torch.dtype):
        super().__init__()
        self.idx = idx
        self.kind = entry["type"]
        self.dtype = dtype
        self.norm1 = _f32_param(width, fill=1.0)
        self.mix = build_mixer(self.kind, entry["mixer"], width, eps, dtype)
        self.mlp = build_ff(entry.get("mlp"), width, dtype)
        self.norm2 = _f32_param(width, fill=1.0) if self.mlp is not None else None

    def cache_shapes(self, block_size: int) -> list:
        if isinstance(self.mix, LatentAttention):
            return [("paged", (block_size, self.mix.rank + self.mix.rot_dim), self.dtype)]
        return self.mix.cache_shapes(block_size)

    def forward(self, x, h1, h2, positions, cache, meta, nxt_w1, nxt_w2, eps):
        """x: f32 stream, updated in place; h1, h2: this layer's two norms of x.
        Returns the two norms of the stream it leaves, taken with the weights
        given (the next layer's, or the final norm's and None)."""
        if isinstance(self.mix, LatentAttention):
            y = self.mix(h1, positions, cache[0], meta)
        else:
            y = self.mix(h1, positions, cache, meta)
        ff, id_w, id_h = None, None, None
        if isinstance(self.mlp, RoutedExperts):
            ff, id_w = self.mlp(h2)
            if self.mlp.identity:
                id_h = h2
            else:
                id_w = None
        elif self.mlp is not None:
            ff = self.mlp(h2)
        return ops.stream_add_rms_norm_pair(x, y, ff, nxt_w1, nxt_w2, eps, self.dtype,
                                            row_scale=id_w, c=id_h)


class ReleraxForCausalLM(nn.Module):
    uses_seq_state = False

    def __init__(self, cfg: ModelConfig):
        super().__init__()
        if get_tp_world_size() != 1:
            raise ValueError("Relerax is not sharded yet; run it with tensor_parallel_size 1")
        hf = cfg.hf_config
        self.cfg = cfg
        dtype = cfg.dtype
        width = cfg.hidden_size
        self.eps = cfg.rms_norm_eps
        self.embed = nn.Parameter(
            torch.empty(cfg.vocab_size, width, dtype=dtype).normal_(0.0, 1.0),
            requires_grad=False)
        self.layers = nn.ModuleList([
            ReleraxLayer(i, e, width, self.eps, dtype) for i, e in enumerate(hf["layers"])])
        self.final_norm = _f32_param(width, fill=1.0)
        self.head = nn.Parameter(
            torch.empty(cfg.vocab_size, width, dtype=dtype).normal_(0.0, width ** -0.5),
            requires_grad=False)
        # set by the test harness to collect the stream after every layer
        self.stream_probe: Optional[list] = None

    # -- cache layout (asked for by the worker) ----------------------------
    @staticmethod
    def _bytes(shape, dtype) -> int:
        n = 1
        for s in shape:
            n *= s
        return n * torch.tensor([], dtype=dtype).element_size()

    def cache_bytes_per_block(self, block_size: int) -> int:
        return max(1, sum(self._bytes(shape, dt) for layer in self.layers
                          for _, shape, dt in layer.cache_shapes(block_size)))

    def state_bytes_per_slot(self) -> int:
        return 0

    def allocate_caches(self, num_blocks: int, block_size: int, num_slots: int,
                        device) -> list:
        """Per layer the paged tensors its mixer names: keys and values
        [blocks, block, kv_heads, dim] for attention, latent rows [blocks,
        block, rank + rot] for latent attention."""
        return [tuple(torch.zeros((num_blocks,) + tuple(shape), dtype=dt, device=device)
                      for _, shape, dt in layer.cache_shapes(block_size))
                for layer in self.layers]

    # -- forward -----------------------------------------------------------
    def forward(self, input_ids, positions, kv_caches, meta: AttnMetadata) -> torch.Tensor:
        x = ops.embedding_scaled(input_ids, self.embed, 1.0)          # f32 [T, W]
        first = self.layers[0]
        h1, h2 = ops.stream_add_rms_norm_pair(x, None, None, first.norm1, first.norm2,
                                              self.eps, self.cfg.dtype)
        last = len(self.layers) - 1
        for i, layer in enumerate(self.layers):
            if i < last:
                w1, w2 = self.layers[i + 1].norm1, self.layers[i + 1].norm2
            else:
                w1, w2 = self.final_norm, None
            h1, h2 = layer(x, h1, h2, positions, kv_caches[i], meta, w1, w2, self.eps)
            if self.stream_probe is not None:
                self.stream_probe.append(x.clone())
        return h1

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return ops.linear(hidden, self.head).float()

    # -- weights -----------------------------------------------------------
    def load_weights(self, weights: dict[str, torch.Tensor]) -> None:
        dtype = self.cfg.dtype
        self.embed.data.copy_(weights["embed"].to(dtype))
        self.head.data.copy_(weights["head"].to(dtype))
        self.final_norm.data.copy_(weights["final.norm"].float())
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            layer.norm1.data.copy_(weights[p + "norm1"].float())
            if isinstance(layer.mix, LatentAttention):
                layer.mix.load(weights[p + "mix.q"], weights[p + "mix.dkv"],
                               weights[p + "mix.dkv.norm"], weights[p + "mix.uk"],
                               weights[p + "mix.uv"], None, weights[p + "mix.o"],
                               gate=weights[p + "mix.g"])
            else:
                layer.mix.load({k[len(p) + 4:]: v for k, v in weights.items()
                                if k.startswith(p + "mix.")})
            if layer.mlp is None:
                continue
            layer.norm2.data.copy_(weights[p + "norm2"].float())
            if isinstance(layer.mlp, RoutedExperts):
                n = layer.mlp.experts
                layer.mlp.load(weights[p + "mlp.router"], weights[p + "mlp.correction"],
                               [weights[f"{p}mlp.e{e}.up"] for e in range(n)],
                               [weights[f"{p}mlp.e{e}.down"] for e in range(n)])
            else:
                layer.mlp.load(weights[p + "mlp.up"], weights[p + "mlp.up.b"],
                               weights[p + "mlp.down"], weights[p + "mlp.down.b"])
