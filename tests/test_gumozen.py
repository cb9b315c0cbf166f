"""Gumozen through the engine against the plain oracle (tests/gumozen_oracle.py).

Every test builds its own small configuration with random weights.  CPU runs
use the reference ops, GPU runs (marked) the HIP kernels; both go through the
engine's request, cache-block and state-slot bookkeeping.
"""

from __future__ import annotations

import math

import pytest
import torch

import gumozen_oracle as oracle
from vllm_tgis_adapter_amd import ops
from vllm_tgis_adapter_amd.engine import EngineConfig, LLMEngine, ModelConfig, SamplingParams
from vllm_tgis_adapter_amd.engine.config import CacheConfig, SchedulerConfig
from vllm_tgis_adapter_amd.models import blocks

CPU = pytest.param("cpu", id="cpu")
GPU = pytest.param("cuda", id="gpu", marks=pytest.mark.gpu)
DEVICES = [CPU, GPU]
F64 = torch.float64
EPS = 1e-5

SCALING = {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 16}


def attn_spec(heads=4, kv_heads=2, dim=8, vdim=12, chunk=7, rot_dims=6, scaling=SCALING,
              base=50.0, diff=0.3):
    rot = {"base": base, "dims": rot_dims}
    if scaling:
        rot["scaling"] = scaling
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "diff": diff,
            "scale": 1.3 / math.sqrt(dim), "mask": {"size": chunk}, "rot": rot}


def rec_spec(heads=3, dim=6, vdim=10):
    return {"heads": heads, "dim": dim, "vdim": vdim}


def latent_spec(heads=3, dim=6, vdim=10, rank=12, q_rank=9, kv_from=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": rank, "q_rank": q_rank,
         "scale": 1.3 / math.sqrt(dim)}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def moe(experts=5, top=2, ff=12):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def make_config(layers=None, width=32, vocab=50):
    if layers is None:
        layers = [("hgrn2", rec_spec(), moe()),
                  ("latent_attention", latent_spec(), moe(3, 1)),
                  ("attention", attn_spec(), moe(4, 3, 8)),
                  ("latent_attention", latent_spec(2, 8, 4, 12, 16, kv_from=1), None),
                  ("attention", attn_spec(2, 2, 6, 6, chunk=11, rot_dims=2, scaling=None), moe())]
    return {"architecture": "Gumozen", "vocab": vocab, "width": width, "norm": {"eps": EPS},
            "layers": [{"type": t, "mixer": m, "mlp": f} for t, m, f in layers]}


def _engine(path, device, dtype="float32", blocks=64, slots=4, block_size=4, eager=True):
    mc = ModelConfig.from_model_arg(path, dtype=dtype)
    return LLMEngine(EngineConfig(
        model_config=mc,
        cache_config=CacheConfig(block_size=block_size, num_gpu_blocks=blocks),
        scheduler_config=SchedulerConfig(max_num_seqs=slots, max_num_batched_tokens=1 << 20),
        device=device, enforce_eager=eager))


def _tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def _feed(engine, rid, tokens, cuts):
    """Feed one request in portions; logits of every position."""
    rows, at = [], 0
    for n in cuts:
        last = at + n == len(tokens)
        rows.append(engine.replay_step([(rid, tokens[at:at + n], list(range(n)))],
                                       [rid] if last else []))
        at += n
    assert at == len(tokens)
    return torch.cat(rows).double().cpu()


def _close(got, want, dtype="float32", what=""):
    tol = 3e-4 if dtype == "float32" else 0.05 * max(1.0, float(want.abs().max()))
    err = float((got - want).abs().max())
    assert err < tol, f"{what} {err}"


@pytest.fixture
def model(tmp_path):
    cfg = make_config()
    w = oracle.random_weights(cfg, seed=1)
    oracle.write_model(str(tmp_path / "m"), cfg, w)
    return cfg, w, str(tmp_path / "m")


# -- each mechanism alone, as the framework's block, in portions --------------


class _Meta:
    """What a mixer reads of the step metadata, for one sequence fed in
    portions through block tables and a state slot of its own."""

    def __init__(self, dev, bs, nblocks, slot):
        self.dev, self.bs, self.slot = dev, bs, slot
        self.blocks = list(range(nblocks - 1, -1, -1))   # scattered on purpose
        self.at = 0

    def step(self, n):
        i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=self.dev)
        s, e = self.at, self.at + n
        self.at = e
        nb = (e + self.bs - 1) // self.bs
        m = type("M", (), {})()
        m.slot_mapping = torch.tensor(
            [self.blocks[p // self.bs] * self.bs + p % self.bs for p in range(s, e)],
            dtype=torch.long, device=self.dev)
        m.seq_start_loc, m.seq_lens, m.state_slots = i32([0, n]), i32([e]), i32([self.slot])
        table = i32([self.blocks[:nb]])
        empty_t, empty = torch.empty((0, 0), dtype=torch.int32, device=self.dev), i32([])
        if n > 1:
            m.num_prefill_tokens, m.num_decode_seqs = n, 0
            m.prefill_block_tables, m.prefill_query_start_loc = table, i32([0, n])
            m.prefill_seq_lens, m.max_prefill_query_len = i32([e]), n
            m.decode_block_tables, m.decode_seq_lens = empty_t, empty
        else:
            m.num_prefill_tokens, m.num_decode_seqs = 0, 1
            m.prefill_block_tables, m.prefill_query_start_loc = empty_t, i32([0])
            m.prefill_seq_lens, m.max_prefill_query_len = empty, 0
            m.decode_block_tables, m.decode_seq_lens = table, i32([e])
        return m, torch.arange(s, e, device=self.dev)


def _run_block(call, cache_shapes, n, dev, cuts, bs=4):
    """``call(rows slice, positions, cache list, meta)`` over n rows fed in
    portions; paged tensors and state slots start dirty."""
    nblocks = (n + bs - 1) // bs + 2
    cache = []
    for kind, shape, dt in cache_shapes:
        lead = nblocks if kind == "paged" else 3
        cache.append(torch.full((lead,) + tuple(shape), 3.0, dtype=dt, device=dev))
    meta = _Meta(dev, bs, nblocks, slot=1)
    outs, at = [], 0
    for k in cuts:
        m, pos = meta.step(k)
        outs.append(call(slice(at, at + k), pos, cache, m).double().cpu())
        at += k
    return torch.cat(outs)


CUTS = [[19], [1] * 19, [2] * 9 + [1], [7, 1, 1, 3, 2, 5], [17, 2]]


@pytest.mark.parametrize("device", DEVICES)
def test_token_shift_alone(device):
    width = 24
    g = torch.Generator().manual_seed(3)
    x = torch.randn(19, width, generator=g)
    w = torch.rand(width, generator=g)
    want = oracle.token_shift(x.double(), w.double())
    mod = blocks.TokenShift(width, torch.float32)
    mod.weight.data.copy_(w)
    mod = mod.to(device)
    for cuts in CUTS:
        got = _run_block(lambda sl, pos, cache, m: mod(x[sl].to(device), cache[0], m),
                         [mod.state_shape()], 19, device, cuts)
        _close(got, want, what=f"cuts {cuts}")


def _attention_weights(spec, width, g):
    nh, ng, d, dv = spec["heads"], spec["kv_heads"], spec["dim"], spec["vdim"]
    sizes = dict(q=(nh * 2 * d, width), k=(ng * 2 * d, width), v=(ng * dv, width),
                 g=(nh, width), o=(width, nh * dv))
    w = {n: torch.randn(r, c, generator=g) / math.sqrt(c) for n, (r, c) in sizes.items()}
    w["q.norm"] = torch.rand(d, generator=g) + 0.5
    w["k.norm"] = torch.rand(d, generator=g) + 0.5
    for n in ("lq1", "lk1", "lq2", "lk2"):
        w[n] = torch.randn(d, generator=g) * 0.4
    return w


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("spec", [
    attn_spec(),
    attn_spec(3, 3, 6, 6, chunk=4, rot_dims=6, scaling=None),   # every dim rotated, heads = kv_heads
    attn_spec(4, 1, 10, 3, chunk=1, rot_dims=2),                # a chunk of one: sees only itself
    attn_spec(2, 2, 16, 20, chunk=0, rot_dims=0),               # no chunks, no rotation
    attn_spec(2, 1, 12, 12, chunk=100, rot_dims=8, diff=0.0,
              scaling={"factor": 8.0, "low": 2.0, "high": 3.0, "original": 40}),
    attn_spec(1, 1, 4, 4, chunk=19, rot_dims=4, diff=0.8),      # the chunk ends with the prompt
])
def test_attention_mixer_alone(device, spec):
    width = 24
    g = torch.Generator().manual_seed(4)
    h = torch.randn(19, width, generator=g)
    w = _attention_weights(spec, width, g)
    nh, ng, d, dv = spec["heads"], spec["kv_heads"], spec["dim"], spec["vdim"]
    want = oracle.differential_attention(
        h.double(), {k: v.double() for k, v in w.items()}, heads=nh, kv_heads=ng, dim=d,
        vdim=dv, scale=spec["scale"], diff=spec["diff"], chunk=spec["mask"]["size"],
        rot=spec["rot"], eps=EPS)
    mod = blocks.DiffAttention(
        width, heads=nh, kv_heads=ng, dim=d, vdim=dv, scale=spec["scale"], diff=spec["diff"],
        eps=EPS, chunk=spec["mask"]["size"], rot_base=spec["rot"]["base"],
        rot_dims=spec["rot"]["dims"], rot_scaling=spec["rot"].get("scaling"),
        dtype=torch.float32)
    mod.load(w)
    mod = mod.to(device)
    for cuts in CUTS:
        got = _run_block(lambda sl, pos, cache, m: mod(h[sl].to(device), pos, cache, m),
                         mod.cache_shapes(4), 19, device, cuts)
        _close(got, want, what=f"cuts {cuts}")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("spec", [rec_spec(), rec_spec(1, 4, 4), rec_spec(4, 16, 3),
                                  rec_spec(2, 5, 33)])
def test_hgrn2_mixer_alone(device, spec):
    width = 24
    g = torch.Generator().manual_seed(5)
    h = torch.randn(19, width, generator=g)
    nh, d, dv = spec["heads"], spec["dim"], spec["vdim"]
    w = {n: torch.randn(r, c, generator=g) / math.sqrt(c) for n, (r, c) in
         dict(q=(nh * d, width), f=(nh * d, width), v=(nh * dv, width),
              o=(width, nh * dv)).items()}
    w["f.b"] = torch.randn(nh * d, generator=g)
    w["lower"] = torch.rand(nh * d, generator=g) * 0.9
    w["norm"] = torch.rand(dv, generator=g) + 0.5
    want = oracle.hgrn2(h.double(), {k: v.double() for k, v in w.items()}, heads=nh, dim=d,
                        vdim=dv, eps=EPS)
    mod = blocks.HGRN2Mixer(width, heads=nh, dim=d, vdim=dv, eps=EPS, dtype=torch.float32)
    mod.load(w)
    mod = mod.to(device)
    for cuts in CUTS:
        got = _run_block(lambda sl, pos, cache, m: mod(h[sl].to(device), pos, cache, m),
                         mod.cache_shapes(4), 19, device, cuts)
        _close(got, want, what=f"cuts {cuts}")


def test_hgrn2_gate_bounds():
    """With the lower bound at 1 nothing is ever written; with the bound at 0
    and a very negative gate the state is the last value: o = v * sum(q)."""
    nh, d, dv, width = 1, 3, 4, 5
    g = torch.Generator().manual_seed(6)
    h = torch.randn(6, width, generator=g).double()
    w = {"q": torch.randn(d, width, generator=g).double(),
         "f": torch.zeros(d, width, dtype=F64), "v": torch.randn(dv, width, generator=g).double(),
         "o": torch.eye(dv, dtype=F64), "norm": torch.ones(dv, dtype=F64),
         "f.b": torch.zeros(d, dtype=F64), "lower": torch.ones(d, dtype=F64)}
    assert float(oracle.hgrn2(h, w, heads=nh, dim=d, vdim=dv, eps=EPS).abs().max()) == 0.0
    w["lower"] = torch.zeros(d, dtype=F64)
    w["f.b"] = torch.full((d,), -60.0, dtype=F64)
    got = oracle.hgrn2(h, w, heads=nh, dim=d, vdim=dv, eps=0.0)
    v = h @ w["v"].T
    qs = oracle.silu(h @ w["q"].T).sum(-1, keepdim=True)
    _close(got, oracle.unit_rms(v * qs, 0.0), what="state = last value")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("spec", [latent_spec(), latent_spec(1, 4, 4, 4, 4),
                                  latent_spec(4, 8, 8, 16, 40), latent_spec(2, 2, 20, 5, 3)])
def test_latent_mixer_alone(device, spec):
    width = 24
    g = torch.Generator().manual_seed(7)
    h = torch.randn(19, width, generator=g)
    nh, d, dv, rank, qr = (spec[k] for k in ("heads", "dim", "vdim", "kv_rank", "q_rank"))
    sizes = {"dq": (qr, width), "uq": (nh * d, qr), "dkv": (rank, width), "uk": (nh * d, rank),
             "uv": (nh * dv, rank), "o": (width, nh * dv)}
    w = {n: torch.randn(a, b, generator=g) / math.sqrt(b) for n, (a, b) in sizes.items()}
    w["dq.norm"] = torch.rand(qr, generator=g) + 0.5
    w["dkv.norm"] = torch.rand(rank, generator=g) + 0.5
    want, _ = oracle.latent_attention(h.double(), {k: v.double() for k, v in w.items()}, None,
                                      heads=nh, dim=d, vdim=dv, scale=spec["scale"], eps=EPS)
    mod = blocks.LatentAttention(
        width, heads=nh, dim=d, rot_dim=0, vdim=dv, rank=rank, scale=spec["scale"], window=0,
        rot_base=10000.0, rot_dims=0, eps=EPS, kv_owner=True, has_sink=False,
        dtype=torch.float32, q_rank=qr)
    mod.load(w["uq"], w["dkv"], w["dkv.norm"], w["uk"], w["uv"], None, w["o"], dq=w["dq"],
             dq_norm=w["dq.norm"])
    mod = mod.to(device)
    for cuts in CUTS:
        got = _run_block(lambda sl, pos, cache, m: mod(h[sl].to(device), pos, cache[0], m),
                         [("paged", (4, rank), torch.float32)], 19, device, cuts)
        _close(got, want, what=f"cuts {cuts}")


@pytest.mark.parametrize("device", DEVICES)
def test_routed_experts_alone(device):
    width = 24
    g = torch.Generator().manual_seed(8)
    h = torch.randn(21, width, generator=g)
    for experts, top, ff in [(5, 2, 12), (1, 1, 8), (4, 4, 6), (12, 1, 10), (3, 2, 16)]:
        router = torch.randn(experts, width, generator=g) / 2
        ex = [(torch.randn(ff, width, generator=g) / 5, torch.randn(ff, width, generator=g) / 5,
               torch.randn(width, ff, generator=g) / 3) for _ in range(experts)]
        want = oracle.routed_gated_ff(h.double(), router.double(),
                                      [tuple(t.double() for t in e) for e in ex], top=top)
        mod = blocks.GatedRoutedExperts(width, experts=experts, top=top, ff=ff,
                                        dtype=torch.float32)
        mod.load(router, [e[0] for e in ex], [e[1] for e in ex], [e[2] for e in ex])
        mod = mod.to(device)
        _close(mod(h.to(device)).double().cpu(), want, what=f"experts {experts} top {top}")
        # the router may be fed the rows the experts' input was rounded from
        _close(mod(h.to(device), router_in=h.to(device)).double().cpu(), want,
               what="router fed separately")


def test_weight_on_the_input_is_not_weight_on_the_output():
    """The gated expert is not linear in its input: weighing the input by s is
    s^2 silu-ish, not s times the plain output."""
    g = torch.Generator().manual_seed(9)
    h = torch.randn(1, 6, generator=g).double()
    ex = [(torch.randn(4, 6, generator=g).double(), torch.randn(4, 6, generator=g).double(),
           torch.randn(6, 4, generator=g).double())]
    router = torch.zeros(1, 6, dtype=F64)         # score 1/2
    got = oracle.routed_gated_ff(h, router, ex, top=1)[0]
    gate, up, down = ex[0]
    x = 0.5 * h[0]
    _close(got, down @ (oracle.silu(gate @ x) * (up @ x)), what="weighted input")
    plain = down @ (oracle.silu(gate @ h[0]) * (up @ h[0]))
    assert float((got - 0.5 * plain).abs().max()) > 1e-3


@pytest.mark.parametrize("device", DEVICES)
def test_grouped_experts_match_oracle(device):
    """The grouped way of running the experts (bf16, sizes in multiples of 128)."""
    width, ff, experts, top = 128, 128, 6, 2
    g = torch.Generator().manual_seed(10)
    bf = torch.bfloat16
    h = torch.randn(37, width, generator=g).to(bf)
    router = (torch.randn(experts, width, generator=g) / 4).to(bf)
    ex = [((torch.randn(ff, width, generator=g) / 11).to(bf),
           (torch.randn(ff, width, generator=g) / 11).to(bf),
           (torch.randn(width, ff, generator=g) / 11).to(bf)) for _ in range(experts)]
    margins = []
    want = oracle.routed_gated_ff(h.double(), router.double(),
                                  [tuple(t.double() for t in e) for e in ex], top=top,
                                  margins=margins)
    keep = [t for t, m in enumerate(margins) if m > 1e-3]
    for grouped in (True, False):
        mod = blocks.GatedRoutedExperts(width, experts=experts, top=top, ff=ff, dtype=bf,
                                        grouped=grouped)
        mod.load(router, [e[0] for e in ex], [e[1] for e in ex], [e[2] for e in ex])
        got = mod.to(device)(h.to(device)).double().cpu()
        _close(got[keep], want[keep], "bfloat16", f"grouped={grouped}")


def test_stepped_frequencies():
    """Short wavelengths keep their frequency, long ones turn ``factor`` times
    slower, the blend between is continuous at both ends."""
    rot = {"base": 100.0, "dims": 16, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0,
                                                  "original": 32}}
    got = blocks.stepped_rotary_frequencies(100.0, 16, rot["scaling"])
    want = oracle.stepped_frequencies(rot)
    plain = oracle.stepped_frequencies({"base": 100.0, "dims": 16})
    assert max(abs(a - b) / b for a, b in zip(got, want)) < 1e-12
    kinds = set()
    for f, p in zip(want, plain):
        wave = 2 * math.pi / p
        if wave < 8:
            assert f == p
            kinds.add("kept")
        elif wave > 32:
            assert abs(f - p / 8.0) < 1e-15
            kinds.add("slowed")
        else:
            assert p / 8.0 <= f <= p
            kinds.add("blended")
    assert kinds == {"kept", "slowed", "blended"}
    assert blocks.stepped_rotary_frequencies(100.0, 16, None) == plain


# -- the whole model through the engine ----------------------------------------


@pytest.mark.parametrize("device", DEVICES)
def test_whole_prompt_and_layers_match_oracle(model, device):
    cfg, w, path = model
    toks = _tokens(23, cfg["vocab"], 2)
    layers = []
    want = oracle.forward(cfg, w, toks, layers)
    eng = _engine(path, device)
    probe = eng.worker.model.stream_probe = []
    got = _feed(eng, "a", toks, [len(toks)])
    _close(got, want, what="logits")
    assert len(probe) == len(layers)
    for i, (a, b) in enumerate(zip(probe, layers)):
        _close(a.double().cpu(), b, what=f"stream after layer {i}")


@pytest.mark.parametrize("device", DEVICES)
def test_decode_and_portions_equal_whole(model, device):
    cfg, w, path = model
    toks = _tokens(31, cfg["vocab"], 3)
    want = oracle.forward(cfg, w, toks)
    eng = _engine(path, device)
    for k, cuts in enumerate([[1] * 31, [2] * 15 + [1], [5, 3, 2, 7, 1, 1, 4, 8], [29, 2],
                              [3] + [1] * 28, [4, 4, 4, 4, 4, 4, 4, 3], [7, 7, 7, 7, 3]]):
        _close(_feed(eng, f"r{k}", toks, cuts), want, what=f"cuts {cuts}")


@pytest.mark.parametrize("device", DEVICES)
def test_long_decode_past_every_chunk(model, device):
    cfg, w, path = model
    toks = _tokens(60, cfg["vocab"], 4)
    want = oracle.forward(cfg, w, toks)
    eng = _engine(path, device)
    _close(_feed(eng, "a", toks, [5] + [1] * 55), want)


@pytest.mark.parametrize("device", DEVICES)
def test_mixed_batch_and_reuse_of_blocks_and_slots(model, device):
    """Unequal requests in one step, portions beside single tokens, requests
    that leave and hand their blocks and state slots to later ones."""
    cfg, w, path = model
    lens = {"a": 26, "b": 9, "c": 17, "d": 30, "e": 12, "f": 21}
    toks = {k: _tokens(n, cfg["vocab"], 10 + i) for i, (k, n) in enumerate(lens.items())}
    want = {k: oracle.forward(cfg, w, t) for k, t in toks.items()}
    # all six need 32 blocks of 4 tokens and six slots; the pool has 22 blocks
    # and 4 slots: the later requests run where finished ones were
    eng = _engine(path, device, blocks=22, slots=4)
    plan = [
        [("a", 7), ("b", 2)],
        [("a", 1), ("b", 5), ("c", 17)],
        [("a", 9), ("b", 1), ("d", 3)],
        [("a", 1), ("b", 1), ("d", 2)],
        [("a", 2), ("d", 1), ("e", 12)],
        [("a", 6), ("d", 24), ("f", 1)],
        [("f", 2)],
        [("f", 18)],
    ]
    at = {k: 0 for k in lens}
    got = {k: [] for k in lens}
    free_before = eng.block_manager.num_free_blocks
    for step in plan:
        entries, end = [], []
        for k, n in step:
            entries.append((k, toks[k][at[k]:at[k] + n], list(range(n))))
            at[k] += n
            if at[k] == lens[k]:
                end.append(k)
        out = eng.replay_step(entries, end).double().cpu()
        row = 0
        for k, n in step:
            got[k].append(out[row:row + n])
            row += n
    assert at == lens
    assert eng.block_manager.num_free_blocks == free_before
    for k in lens:
        _close(torch.cat(got[k]), want[k], what=k)


def test_a_request_may_sit_out_steps(model):
    """A request left out of a step goes on later from the state it left."""
    cfg, w, path = model
    ta, tb = _tokens(14, cfg["vocab"], 40), _tokens(11, cfg["vocab"], 41)
    eng = _engine(path, "cpu")
    ga, gb = [], []
    ga.append(eng.replay_step([("a", ta[:6], list(range(6)))], []))
    gb.append(eng.replay_step([("b", tb[:4], list(range(4)))], []))
    gb.append(eng.replay_step([("b", tb[4:5], [0])], []))
    out = eng.replay_step([("a", ta[6:7], [0]), ("b", tb[5:], list(range(6)))], ["b"])
    ga.append(out[:1])
    gb.append(out[1:])
    ga.append(eng.replay_step([("a", ta[7:], list(range(7)))], ["a"]))
    _close(torch.cat(ga).double(), oracle.forward(cfg, w, ta), what="a")
    _close(torch.cat(gb).double(), oracle.forward(cfg, w, tb), what="b")


VARIANTS = {
    "no_ff_one_head": [("attention", attn_spec(1, 1, 8, 8, chunk=3, rot_dims=8), None),
                       ("hgrn2", rec_spec(1, 4, 4), None),
                       ("latent_attention", latent_spec(1, 4, 4, 4, 4), None)],
    "attention_only": [("attention", attn_spec(6, 3, 4, 2, chunk=2, rot_dims=2, scaling=None),
                        moe(2, 1, 6)),
                       ("attention", attn_spec(2, 2, 12, 5, chunk=50, rot_dims=12, diff=0.6),
                        moe(3, 3, 8))],
    "recurrent_only": [("hgrn2", rec_spec(2, 10, 3), moe(4, 4, 5)),
                       ("hgrn2", rec_spec(5, 2, 6), None)],
    "shared_latents": [("latent_attention", latent_spec(2, 10, 3, 7, 5), moe(4, 2, 5)),
                       ("latent_attention", latent_spec(5, 2, 6, 7, 20, kv_from=0), moe(1, 1, 9)),
                       ("latent_attention", latent_spec(1, 6, 6, 7, 7, kv_from=0), None),
                       ("latent_attention", latent_spec(3, 4, 4, 9, 2), None),
                       ("latent_attention", latent_spec(3, 4, 4, 9, 2, kv_from=3), None)],
}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("variant", sorted(VARIANTS))
def test_other_shapes(tmp_path, device, variant):
    cfg = make_config(VARIANTS[variant], width=20, vocab=31)
    w = oracle.random_weights(cfg, seed=5)
    oracle.write_model(str(tmp_path / "v"), cfg, w)
    toks = _tokens(22, cfg["vocab"], 6)
    want = oracle.forward(cfg, w, toks)
    eng = _engine(str(tmp_path / "v"), device, block_size=8)
    _close(_feed(eng, "a", toks, [22]), want, what="whole")
    _close(_feed(eng, "b", toks, [3, 2, 9, 1, 1, 6]), want, what="portions")


@pytest.mark.parametrize("device", DEVICES)
def test_bf16_stays_near_oracle(model, device):
    cfg, w, path = model
    toks = _tokens(25, cfg["vocab"], 7)
    margins = []
    want = oracle.forward(cfg, w, toks, margins_out=margins)
    # a router's close call may go the other way in bf16: those positions prove
    # nothing (later positions see them only through caches and state)
    first_bad = next((t for t in range(len(toks)) if min(m[t] for m in margins) < 2e-3),
                     len(toks))
    assert first_bad > 5
    eng = _engine(path, device, dtype="bfloat16")
    got = _feed(eng, "a", toks, [11, 1, 1, 12])
    _close(got[:first_bad], want[:first_bad], "bfloat16")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_matrix_core_shapes(tmp_path, dtype):
    """Head sizes the matrix-core attention kernels take, long enough for
    several key tiles, chunks that end inside a tile; a latent of a size the
    matrix-core latent kernel takes; experts of a size the grouped product
    takes (bf16 runs them grouped, f32 stacked)."""
    layers = [("attention", attn_spec(2, 1, 128, 128, chunk=70, rot_dims=64), moe(5, 2, 128)),
              ("latent_attention", latent_spec(4, 32, 48, 64, 96), None),
              ("hgrn2", rec_spec(2, 64, 64), None),
              ("attention", attn_spec(4, 2, 64, 64, chunk=33, rot_dims=64, scaling=None), None),
              ("latent_attention", latent_spec(2, 64, 64, 64, 32, kv_from=1), None)]
    cfg = make_config(layers, width=128, vocab=40)
    w = oracle.random_weights(cfg, seed=8)
    oracle.write_model(str(tmp_path / "m"), cfg, w)
    toks = _tokens(150, cfg["vocab"], 9)
    margins = []
    want = oracle.forward(cfg, w, toks, margins_out=margins)
    first_bad = len(toks) if dtype == "float32" else next(
        (t for t in range(len(toks)) if min(m[t] for m in margins) < 2e-3), len(toks))
    assert first_bad > 20
    eng = _engine(str(tmp_path / "m"), "cuda", dtype=dtype, blocks=40, block_size=16)
    assert eng.worker.model.layers[0].mlp.grouped == (dtype == "bfloat16")
    _close(_feed(eng, "a", toks, [150])[:first_bad], want[:first_bad], dtype, "whole")
    _close(_feed(eng, "b", toks, [70, 3, 40, 2] + [1] * 35)[:first_bad], want[:first_bad],
           dtype, "portions")


@pytest.mark.gpu
def test_captured_decode_steps_match_eager(model):
    cfg, w, path = model
    prompts = {k: _tokens(n, cfg["vocab"], 20 + i) for i, (k, n) in
               enumerate({"a": 9, "b": 4, "c": 13}.items())}

    def generate(eager):
        eng = _engine(path, "cuda", eager=eager)
        for k, t in prompts.items():
            eng.add_request(k, None, list(t), SamplingParams(temperature=0.0, max_tokens=12))
        out = {}
        while eng.has_unfinished():
            for o in eng.step():
                if o.finished:
                    out[o.request_id] = list(o.outputs[0].token_ids)
        return out, eng

    eager, _ = generate(True)
    graphs, eng = generate(False)
    assert eng.worker.graph_runner is not None and eng.worker.graph_runner.graphs
    assert eager == graphs


# -- keys far away, at page borders, just inside and outside a chunk ------------


def _spiky_attention(chunk, ctx, spike_at, n_new, device, bs=4, dim=8, dtype=torch.float32):
    """One head; every key is small noise but the one at ``spike_at``, which
    the last query points at; its value is all 100.  Returns the last query's
    output through the op, and the same from the definition."""
    g = torch.Generator().manual_seed(ctx * 31 + spike_at)
    k = torch.randn(ctx, 1, dim, generator=g) * 0.05
    v = torch.randn(ctx, 1, dim, generator=g) * 0.05
    q = torch.randn(n_new, 1, dim, generator=g) * 0.05
    direction = torch.ones(dim) / math.sqrt(dim)
    k[spike_at, 0] = 6.0 * direction
    v[spike_at, 0] = 100.0
    q[-1, 0] = 6.0 * direction
    k, v, q = k.to(dtype), v.to(dtype), q.to(dtype)
    nb = (ctx + bs - 1) // bs
    table = list(range(nb - 1, -1, -1))
    kc = torch.zeros(nb, bs, 1, dim, dtype=dtype)
    vc = torch.zeros(nb, bs, 1, dim, dtype=dtype)
    for p in range(ctx):
        kc[table[p // bs], p % bs] = k[p]
        vc[table[p // bs], p % bs] = v[p]
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=device)
    out = torch.empty(n_new, 1, dim, device=device)
    if n_new > 1:
        ops.chunk_attention_prefill(q.to(device), kc.to(device), vc.to(device), i32([table]),
                                    i32([0, n_new]), i32([ctx]), 1.0, n_new, chunk, out=out)
    else:
        ops.chunk_attention_decode(q.to(device), kc.to(device), vc.to(device), i32([table]),
                                   i32([ctx]), 1.0, chunk, out=out)
    i = ctx - 1
    lo = (i // chunk) * chunk if chunk else 0
    s = (k[lo:ctx, 0].double() @ q[-1, 0].double())
    e = torch.exp(s - s.max())
    want = (e / e.sum()) @ v[lo:ctx, 0].double()
    return out[-1, 0].double().cpu(), want


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("n_new", [1, 2, 7])
@pytest.mark.parametrize("chunk,ctx", [(6, 30), (6, 31), (8, 8), (8, 9), (16, 200), (0, 200),
                                       (5, 21), (64, 130), (7, 300)])
def test_chunk_edge_and_far_keys(device, n_new, chunk, ctx):
    first = ((ctx - 1) // chunk) * chunk if chunk else 0
    places = {0, ctx - 1, first, first - 1, first + 1}
    places |= {p for p in (3, 4, 7, 8) if p < ctx}            # page borders
    for at in sorted(p for p in places if 0 <= p < ctx):
        got, want = _spiky_attention(chunk, ctx, at, min(n_new, ctx), device)
        seen = at >= first
        assert (float(want.abs().max()) > 50.0) == seen       # the spike decides the output
        assert float((got - want).abs().max()) < 1e-3, f"spike at {at}"


@pytest.mark.gpu
@pytest.mark.parametrize("n_new", [1, 5, 300])
@pytest.mark.parametrize("chunk,ctx", [(64, 130), (100, 700), (0, 700), (257, 600), (128, 512)])
def test_chunk_edge_and_far_keys_on_matrix_cores(n_new, chunk, ctx):
    """The same on the bf16 matrix-core kernels (key size 128)."""
    first = ((ctx - 1) // chunk) * chunk if chunk else 0
    places = {0, ctx - 1, first, first - 1, first + 1, 63, 64, 15, 16}
    for at in sorted(p for p in places if 0 <= p < ctx):
        got, want = _spiky_attention(chunk, ctx, at, min(n_new, ctx), "cuda", bs=16, dim=128,
                                     dtype=torch.bfloat16)
        assert (float(want.abs().max()) > 50.0) == (at >= first)
        assert float((got - want).abs().max()) < 0.5, f"spike at {at}"


@pytest.mark.parametrize("device", DEVICES)
def test_differential_maps_cancel(device):
    """With both maps equal and lambda = 1 the head's output is zero before
    the norm: the norm's eps keeps it zero instead of blowing it up."""
    a = torch.randn(3, 1, 2, 8).repeat(1, 2, 1, 1).to(device)
    out = ops.diff_combine(a, 1.0, 0.7, 1e-6, None, torch.float32)
    assert float(out.abs().max()) < 1e-12
    out = ops.diff_combine(a, 0.0, 0.7, 0.0, None, torch.float32).view(3, 2, 8)
    want = oracle.unit_rms(a[:, 0].double().cpu(), 0.0) * 0.7
    _close(out.double().cpu(), want, what="lambda 0")


# -- generation through the engine's own entry point --------------------------


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_matches_oracle(model, device):
    cfg, w, path = model
    prompts = {"a": _tokens(7, cfg["vocab"], 30), "b": _tokens(15, cfg["vocab"], 31),
               "c": _tokens(2, cfg["vocab"], 32)}
    steps = 10
    eng = _engine(path, device)
    for k, t in prompts.items():
        eng.add_request(k, None, list(t), SamplingParams(temperature=0.0, max_tokens=steps))
    got = {}
    while eng.has_unfinished():
        for o in eng.step():
            if o.finished:
                got[o.request_id] = list(o.outputs[0].token_ids)
    for k, t in prompts.items():
        seq = list(t)
        for j in range(steps):
            logits = oracle.forward(cfg, w, seq)[-1]
            top2 = torch.topk(logits, 2).values
            if float(top2[0] - top2[1]) < 1e-3:      # a close call proves nothing
                break
            nxt = int(torch.argmax(logits))
            assert got[k][j] == nxt, f"{k}: token {j}"
            seq.append(got[k][j])


def test_registry_and_cache_layout(tmp_path):
    cfg = make_config()
    oracle.write_model(str(tmp_path / "m"), cfg, oracle.random_weights(cfg, seed=2))
    mc = ModelConfig.from_model_arg(str(tmp_path / "m"), dtype="float32")
    assert mc.architecture == "gumozen" and mc.num_layers == 5 and mc.vocab_size == 50
    from vllm_tgis_adapter_amd.models import get_model, native_extensions

    assert native_extensions(mc) == ["_C_seq", "_C_lat"]
    m = get_model(mc)
    assert m.uses_seq_state
    caches = m.allocate_caches(3, 4, 2, "cpu")
    shapes = [[tuple(c.shape) for c in cs] for cs in caches]
    assert shapes[0] == [(2, 3, 10, 6), (2, 32)]                 # recurrent state, shift row
    assert shapes[1] == [(3, 4, 12), (2, 32)]                    # latent rows, shift row
    assert shapes[2] == [(3, 4, 4, 8), (3, 4, 2, 12), (2, 32)]   # keys of both maps, values
    assert shapes[3] == [(3, 4, 12), (2, 32)]                    # the borrowed rows
    assert caches[3][0] is caches[1][0]
    assert m.cache_bytes_per_block(4) == 4 * (4 * 12 + 4 * (4 * 8 + 2 * 12) + 4 * (4 * 6 + 2 * 6))


def test_config_errors(tmp_path):
    from vllm_tgis_adapter_amd.models.gumozen import model_config_from_json

    bad = make_config([("latent_attention", latent_spec(kv_from=0), None)])
    with pytest.raises(ValueError):
        model_config_from_json("x", bad)
    bad = make_config([("latent_attention", latent_spec(rank=8), None),
                       ("latent_attention", latent_spec(rank=12, kv_from=0), None)])
    with pytest.raises(ValueError):
        model_config_from_json("x", bad)
    bad = make_config([("conv", {}, None)])
    with pytest.raises(ValueError):
        model_config_from_json("x", bad)


def test_served_from_command_line_flags(tmp_path):
    """A model directory given as --model goes through the server's flag
    parsing into the async engine and streams greedy tokens equal to the
    oracle's, concurrent requests included."""
    import asyncio

    from vllm_tgis_adapter_amd.__main__ import parse_args
    from vllm_tgis_adapter_amd.engine.async_engine import AsyncLLMEngine
    from vllm_tgis_adapter_amd.tgis_utils.args import engine_config_from_args

    cfg = make_config(vocab=300)    # room for the byte-level test tokenizer
    w = oracle.random_weights(cfg, seed=5)
    oracle.write_model(str(tmp_path / "served"), cfg, w)
    args = parse_args(["--model", str(tmp_path / "served"), "--dtype", "float32",
                       "--max-num-seqs", "2", "--num-gpu-blocks", "64", "--block-size", "8",
                       "--device", "cpu"])
    engine = AsyncLLMEngine(engine_config_from_args(args))
    prompts = {"x": _tokens(12, 300, 61), "y": _tokens(5, 300, 62), "z": _tokens(9, 300, 63)}

    async def one(rid):
        last = None
        async for out in engine.generate(
                {"prompt_token_ids": prompts[rid]},
                SamplingParams(temperature=0.0, max_tokens=5), request_id=rid):
            last = out
        return rid, list(last.outputs[0].token_ids)

    async def main():
        return dict(await asyncio.gather(*[one(r) for r in prompts]))

    try:
        got = asyncio.run(main())
    finally:
        engine.shutdown()
    eos = engine.engine.eos_token_id
    for rid, p in prompts.items():
        seq = list(p)
        for j in range(5):
            logits = oracle.forward(cfg, w, seq)[-1]
            top2 = torch.topk(logits, 2).values
            if float(top2[0] - top2[1]) < 1e-3:
                break
            seq.append(int(logits.argmax()))
            assert got[rid][j] == seq[-1], rid
            if seq[-1] == eos:
                break
