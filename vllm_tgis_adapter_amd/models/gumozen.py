"""Gumozen: a decoder-only model with an f32 residual stream whose sublayers
read the stream itself and are normed on the way out,

    x <- x + ls1 * norm1(mixer(shift(x))),   x <- x + ls2 * norm2(ff(x)),

with RMS norms (plain weight), per-channel layer scales ls*, and a token shift
in front of every mixer: shift(x)_t = x_t + (x_(t-1) - x_t) * w, the previous
row of the stream being part of a sequence's state in every layer.  The
embedding output is RMS-normed before the first layer.  The mixer of a layer
is one of

  attention         differential grouped-query attention (two softmax maps per
                    head over the same values, combined as a_1 - lam a_2 and
                    normed), per-head query/key norm, rotary positions in the
                    half-split layout with piecewise frequency scaling, a
                    chunk mask, a per-head sigmoid gate
  hgrn2             a gated linear recurrence with a matrix state per head
  latent_attention  causal attention over one cached latent row per token,
                    without positions; queries go through a latent of their
                    own; a layer may read the rows of an earlier layer
                    (``kv_from``) with its own up-projections

and the feed-forward is a mixture of small gated experts behind a sigmoid
router, or absent.  The head is the final RMS norm and a linear map.

Sizes and constants all come from config.json:

  vocab, width, norm.eps, layers[i] = {type, mixer{...}, mlp{...} | null}
  attention:  heads, kv_heads, dim, vdim, scale, diff, mask.size, rot{base, dims,
              scaling{factor, low, high, original}}
  hgrn2:      heads, dim, vdim
  latent:     heads, dim, vdim, kv_rank, q_rank, scale, kv_from?
  mlp:        kind "moe", expert.ff, router{experts, top}

Tensors: embed, embed.norm, final.norm, head, l<i>.{norm1, norm2, ls1, ls2,
shift}, l<i>.mix.* (per mixer, see models/blocks.py), l<i>.mlp.{router,
e<j>.gate, e<j>.up, e<j>.down}.
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
    DiffAttention,
    GatedRoutedExperts,
    HGRN2Mixer,
    LatentAttention,
    TokenShift,
    _f32_param,
)

# positions are unbounded in this design; the default bounds block tables and
# capture buffers and can be raised with --max-model-len
_DEFAULT_MAX_LEN = 32768

MIXERS = ("attention", "hgrn2", "latent_attention")


def build_mixer(kind: str, m: dict, width: int, eps: float, dtype: torch.dtype):
    if kind == "attention":
        rot = m.get("rot") or {}
        dim = int(m["dim"])
        return DiffAttention(
            width, heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])),
            dim=dim, vdim=int(m.get("vdim", dim)), scale=float(m["scale"]),
            diff=float(m["diff"]), eps=eps, chunk=int((m.get("mask") or {}).get("size") or 0),
            rot_base=float(rot.get("base", 10000.0)), rot_dims=int(rot.get("dims", 0)),
            rot_scaling=rot.get("scaling"), head_gate=True, dtype=dtype)
    if kind == "hgrn2":
        return HGRN2Mixer(width, heads=int(m["heads"]), dim=int(m["dim"]),
                          vdim=int(m["vdim"]), eps=eps, dtype=dtype)
    if kind == "latent_attention":
        return LatentAttention(
            width, heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=0,
            vdim=int(m["vdim"]), rank=int(m["kv_rank"]), scale=float(m["scale"]),
            window=0, rot_base=10000.0, rot_dims=0, eps=eps,
            kv_owner=m.get("kv_from") is None, has_sink=False, dtype=dtype,
            two_term_weights=True, q_rank=int(m.get("q_rank") or 0))
    raise ValueError(f"unknown mixer type {kind!r}")


def build_ff(mlp: Optional[dict], width: int, dtype: torch.dtype):
    if mlp is None:
        return None
    if mlp.get("kind", "moe") != "moe":
        raise ValueError(f"unknown feed-forward kind {mlp.get('kind')!r}")
    r = mlp["router"]
    return GatedRoutedExperts(width, experts=int(r["experts"]), top=int(r["top"]),
                              ff=int(mlp["expert"]["ff"]), dtype=dtype)


def _check_layers(layers: list) -> None:
    for i, e in enumerate(layers):
        if e.get("type") not in MIXERS:
            raise ValueError(f"layer {i}: unknown mixer type {e.get('type')!r}")
        j = e["mixer"].get("kv_from") if e["type"] == "latent_attention" else None
        if j is None:
            continue
        j = int(j)
        if not (0 <= j < i) or layers[j].get("type") != "latent_attention" \
                or layers[j]["mixer"].get("kv_from") is not None \
                or int(layers[j]["mixer"]["kv_rank"]) != int(e["mixer"]["kv_rank"]):
            raise ValueError(f"layer {i}: kv_from must name an earlier latent-attention "
                             "layer with a latent of its own and of the same rank")


def model_config_from_json(model: str, hf: dict) -> ModelConfig:
    layers = hf["layers"]
    _check_layers(layers)
    att = [e["mixer"] for e in layers if e["type"] == "attention"]
    return ModelConfig(
        model=model,
        architecture="gumozen",
        vocab_size=int(hf["vocab"]),
        hidden_size=int(hf["width"]),
        intermediate_size=max((int(e["mlp"]["expert"]["ff"]) for e in layers if e.get("mlp")),
                              default=0),
        num_layers=len(layers),
        num_heads=max(int(e["mixer"]["heads"]) for e in layers),
        num_kv_heads=max((int(a.get("kv_heads", a["heads"])) for a in att), default=1),
        head_dim=max((int(a["dim"]) for a in att), default=1),
        rope_theta=0.0,
        rms_norm_eps=float((hf.get("norm") or {}).get("eps", 1e-5)),
        max_model_len=int(hf.get("max_len", _DEFAULT_MAX_LEN)),
        tie_word_embeddings=False,
        dtype=torch.bfloat16,
        # num_experts stays 0: that field describes the mixtral expert layout;
        # the routed layers here are shape-static
        hf_config=hf,
    )


def native_extensions(cfg: ModelConfig) -> list[str]:
    """Stream ops, token shift, norm + rotation + cache write, chunk-masked
    attention of any shape, the recurrence, gates and router live in the
    sequence extension; latent attention has its own; an attention mixer whose
    shape the matrix-core kernels take needs the attention extension too."""
    need = ["_C_seq"]
    layers = cfg.hf_config["layers"]
    if any(e.get("type") == "latent_attention" for e in layers):
        need.append("_C_lat")
    for e in layers:
        if e.get("type") != "attention":
            continue
        m = e["mixer"]
        dim = int(m["dim"])
        if ops.chunk_attention_uses_matrix_cores(
                cfg.dtype, int(m["heads"]), int(m.get("kv_heads", m["heads"])), dim,
                int(m.get("vdim", dim))):
            need.append("_C_attn")
            break
    return need


class GumozenLayer(nn.Module):
    def __init__(self, idx: int, entry: dict, width: int, eps: float, dtype: torch.dtype):
        super().__init__()
        self.idx = idx
        self.kind = entry["type"]
        self.dtype = dtype
        self.eps = eps
        self.shift = TokenShift(width, dtype)
        self.mix = build_mixer(self.kind, entry["mixer"], width, eps, dtype)
        kv_from = entry["mixer"].get("kv_from") if self.kind == "latent_attention" else None
        self.kv_from = None if kv_from is None else int(kv_from)
        self.norm1 = _f32_param(width, fill=1.0)
        self.ls1 = _f32_param(width, fill=1.0)
        self.mlp = build_ff(entry.get("mlp"), width, dtype)
        if self.mlp is not None:
            self.norm2 = _f32_param(width, fill=1.0)
            self.ls2 = _f32_param(width, fill=1.0)

    def cache_shapes(self, block_size: int) -> list:
        """The mixer's tensors (a layer that reads another layer's latent rows
        names none), then the token shift's row."""
        if isinstance(self.mix, LatentAttention):
            own = ([("paged", (block_size, self.mix.rank), self.dtype)]
                   if self.kv_from is None else [])
        else:
            own = self.mix.cache_shapes(block_size)
        return own + [self.shift.state_shape()]

    def forward(self, x, positions, cache, meta):
        """x: f32 stream, updated in place.  cache: the mixer's tensors (for a
        latent layer the rows it reads, its own or its owner's), then the
        token shift's state."""
        h = self.shift(x, cache[-1], meta)
        if isinstance(self.mix, LatentAttention):
            y = self.mix(h, positions, cache[0], meta)
        else:
            y = self.mix(h, positions, cache[:-1], meta)
        if self.mlp is None:
            ops.stream_add_rms_norm(x, y, self.norm1, self.eps, 1.0, layer_scale=self.ls1)
            return
        h = ops.stream_add_rms_norm(x, y, self.norm1, self.eps, 1.0, layer_scale=self.ls1,
                                    cast_dtype=self.dtype)
        # the router reads the f32 stream itself, the experts its rounded copy
        ops.stream_add_rms_norm(x, self.mlp(h, router_in=x), self.norm2, self.eps, 1.0,
                                layer_scale=self.ls2)


class GumozenForCausalLM(nn.Module):
    uses_seq_state = True

    def __init__(self, cfg: ModelConfig):
        super().__init__()
        if get_tp_world_size() != 1:
            raise ValueError("Gumozen is not sharded yet; run it with tensor_parallel_size 1")
        hf = cfg.hf_config
        _check_layers(hf["layers"])
        self.cfg = cfg
        dtype = cfg.dtype
        width = cfg.hidden_size
        self.eps = cfg.rms_norm_eps
        self.embed = nn.Parameter(
            torch.empty(cfg.vocab_size, width, dtype=dtype).normal_(0.0, 1.0),
            requires_grad=False)
        self.embed_norm = _f32_param(width, fill=1.0)
        self.layers = nn.ModuleList([
            GumozenLayer(i, e, width, self.eps, dtype) for i, e in enumerate(hf["layers"])])
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
                          for kind, shape, dt in layer.cache_shapes(block_size)
                          if kind == "paged"))

    def state_bytes_per_slot(self) -> int:
        return sum(self._bytes(shape, dt) for layer in self.layers
                   for kind, shape, dt in layer.cache_shapes(1) if kind == "slot")

    def allocate_caches(self, num_blocks: int, block_size: int, num_slots: int,
                        device) -> list:
        """Per layer the tensors it names, paged ones [blocks, ...] and
        per-sequence ones [slots, ...]; a latent layer with ``kv_from`` gets
        its owner's rows in front."""
        out = []
        for layer in self.layers:
            entry = []
            if layer.kv_from is not None:
                entry.append(out[layer.kv_from][0])
            for kind, shape, dt in layer.cache_shapes(block_size):
                lead = num_blocks if kind == "paged" else max(num_slots, 1)
                entry.append(torch.zeros((lead,) + tuple(shape), dtype=dt, device=device))
            out.append(tuple(entry))
        return out

    # -- forward -----------------------------------------------------------
    def forward(self, input_ids, positions, kv_caches, meta: AttnMetadata) -> torch.Tensor:
        e = torch.nn.functional.embedding(input_ids, self.embed)
        x = torch.zeros(e.shape, dtype=torch.float32, device=e.device)   # f32 stream
        ops.stream_add_rms_norm(x, e, self.embed_norm, self.eps, 1.0)
        for i, layer in enumerate(self.layers):
            layer(x, positions, kv_caches[i], meta)
            if self.stream_probe is not None:
                self.stream_probe.append(x.clone())
        return ops.rms_norm_stream(x, self.final_norm, self.eps, 0.0, self.cfg.dtype)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return ops.linear(hidden, self.head).float()

    # -- weights -----------------------------------------------------------
    @staticmethod
    def _sub(weights: dict, prefix: str) -> dict:
        return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}

    def load_weights(self, weights: dict[str, torch.Tensor]) -> None:
        dtype = self.cfg.dtype
        self.embed.data.copy_(weights["embed"].to(dtype))
        self.embed_norm.data.copy_(weights["embed.norm"].float())
        self.head.data.copy_(weights["head"].to(dtype))
        self.final_norm.data.copy_(weights["final.norm"].float())
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            layer.shift.weight.data.copy_(weights[p + "shift"].float())
            layer.norm1.data.copy_(weights[p + "norm1"].float())
            layer.ls1.data.copy_(weights[p + "ls1"].float())
            t = self._sub(weights, p + "mix.")
            if isinstance(layer.mix, LatentAttention):
                own = layer.kv_from is None
                layer.mix.load(t["uq"], t["dkv"] if own else None,
                               t["dkv.norm"] if own else None, t["uk"], t["uv"], None,
                               t["o"], dq=t["dq"], dq_norm=t["dq.norm"])
            else:
                layer.mix.load(t)
            if layer.mlp is None:
                continue
            layer.norm2.data.copy_(weights[p + "norm2"].float())
            layer.ls2.data.copy_(weights[p + "ls2"].float())
            n = layer.mlp.experts
            layer.mlp.load(weights[p + "mlp.router"],
                           [weights[f"{p}mlp.e{e}.gate"] for e in range(n)],
                           [weights[f"{p}mlp.e{e}.up"] for e in range(n)],
                           [weights[f"{p}mlp.e{e}.down"] for e in range(n)])
