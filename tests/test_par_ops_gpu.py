"""HIP kernels of the two-norm residual op, rotation + cache write (half-split
and interleaved pairs), windowed attention with a sink, output gates, squared
relu, the expert router and the expert combine against the plain-PyTorch
reference ops, on sizes that hit vector and scalar paths."""

import pytest
import torch

from vllm_tgis_adapter_amd import ops
from vllm_tgis_adapter_amd.ops import reference as ref

pytestmark = pytest.mark.gpu

DEV = "cuda"
DTYPES = [torch.float32, torch.bfloat16]


def _close(a, b, dtype, what=""):
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    a, b = a.float().cpu(), b.float().cpu()
    assert a.shape == b.shape, what
    if a.numel() == 0:
        return
    scale = max(1.0, float(b.abs().max()))
    err = float((a - b).abs().max()) / scale
    assert err < tol, f"{what}: {err}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [6, 96, 250, 1024, 5120])
def test_two_norm_residual(dtype, width):
    g = torch.Generator().manual_seed(1)
    rows = 5
    x = torch.randn(rows, width, generator=g) * 3
    a = torch.randn(rows, width, generator=g).to(dtype)
    b = torch.randn(rows, width, generator=g).to(dtype)
    c = torch.randn(rows, width, generator=g).to(dtype)
    rs = torch.rand(rows, generator=g)
    w1 = torch.rand(width, generator=g) + 0.5
    w2 = torch.rand(width, generator=g) + 0.5
    cases = [
        (None, None, None, None, w1, w2),
        (a, None, None, None, w1, w2),
        (a, b, None, None, w1, None),
        (a, b, rs, c, w1, w2),
        (a, None, rs, c, None, None),
    ]
    for aa, bb, rr, cc, u1, u2 in cases:
        xr = x.clone()
        h1r, h2r = ref.stream_add_rms_norm_pair(xr, aa, bb, rr, cc, u1, u2, 1e-5, dtype)
        xg = x.clone().to(DEV)
        mv = lambda t: None if t is None else t.to(DEV)
        h1g, h2g = ops.stream_add_rms_norm_pair(xg, mv(aa), mv(bb), mv(u1), mv(u2), 1e-5,
                                                dtype, row_scale=mv(rr), c=mv(cc))
        _close(xg, xr, torch.float32, "stream")
        for hg, hr in ((h1g, h1r), (h2g, h2r)):
            assert (hg is None) == (hr is None)
            if hr is not None:
                _close(hg, hr, dtype, "norm")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("interleaved", [False, True])
@pytest.mark.parametrize("heads,kv_heads,dim,rot", [(4, 2, 24, 12), (3, 3, 64, 64),
                                                   (8, 1, 128, 32), (2, 2, 10, 0)])
def test_rotation_and_cache_write(dtype, interleaved, heads, kv_heads, dim, rot):
    g = torch.Generator().manual_seed(2)
    t, bs, nblocks = 9, 4, 6
    wide = torch.randn(t, (heads + kv_heads) * dim + 8, generator=g).to(dtype)
    q = wide[:, :heads * dim].view(t, heads, dim)
    k = wide[:, heads * dim:(heads + kv_heads) * dim].view(t, kv_heads, dim)
    pos = torch.tensor([0, 1, 2, 3, 700, 701, 30000, 5, 6])
    inv = torch.tensor([10000.0 ** (-2.0 * i / max(rot, 2)) for i in range(max(rot, 2) // 2)])
    slots = torch.tensor([3, 2, 1, 0, 11, 12, 23, -1, 17])
    kc_r = torch.zeros(nblocks, bs, kv_heads, dim, dtype=dtype)
    vc_r = torch.zeros_like(kc_r)
    q_r = ref.rope_kv_cache_write(q, k, k, pos, inv, rot, interleaved, 1.07, kc_r, vc_r, slots)
    kc_g, vc_g = torch.zeros_like(kc_r).to(DEV), torch.zeros_like(kc_r).to(DEV)
    wd = wide.to(DEV)
    qd = wd[:, :heads * dim].view(t, heads, dim)
    kd = wd[:, heads * dim:(heads + kv_heads) * dim].view(t, kv_heads, dim)
    q_g = ops.rope_kv_cache_write(qd, kd, kd, pos.to(DEV), inv.to(DEV), rot, interleaved,
                                  1.07, kc_g, vc_g, slots.to(DEV))
    _close(q_g, q_r, dtype, "q")
    _close(kc_g, kc_r, dtype, "k cache")
    _close(vc_g, vc_r, dtype, "v cache")

    # the in-place rotation of a slice of each head and the latent row writer
    x = torch.randn(t, heads, dim + 6, generator=g).to(dtype)
    xr = x.clone()
    ref.rope_partial(xr, pos, inv, 6, rot, interleaved, 0.9)
    xg = x.clone().to(DEV)
    ops.rope_partial(xg, pos.to(DEV), inv.to(DEV), 6, rot, interleaved, 0.9)
    _close(xg, xr, dtype, "rope_partial")
    rank = 20
    dkv = torch.randn(t, rank + dim, generator=g).to(dtype)
    nw = torch.rand(rank, generator=g) + 0.5
    lc_r = torch.zeros(nblocks, bs, rank + dim, dtype=dtype)
    ref.latent_kv_write(dkv, nw, 1e-5, pos, inv, rot, lc_r, slots, interleaved, 1.07)
    lc_g = torch.zeros_like(lc_r).to(DEV)
    ops.latent_kv_write(dkv.to(DEV), nw.to(DEV), 1e-5, pos.to(DEV), inv.to(DEV), rot, lc_g,
                        slots.to(DEV), interleaved, 1.07)
    _close(lc_g, lc_r, dtype, "latent rows")


def _paged(ctxs, bs, kv_heads, dim, vdim, dtype, g, spare=3):
    """Caches filled for sequences of the given lengths, blocks handed out in
    a scrambled order."""
    nb = sum((c + bs - 1) // bs for c in ctxs) + spare
    perm = torch.randperm(nb, generator=g).tolist()
    kc = torch.randn(nb, bs, kv_heads, dim, generator=g).to(dtype)
    vc = torch.randn(nb, bs, kv_heads, vdim, generator=g).to(dtype)
    width = max((c + bs - 1) // bs for c in ctxs)
    bt = torch.zeros(len(ctxs), width, dtype=torch.int32)
    for i, c in enumerate(ctxs):
        n = (c + bs - 1) // bs
        bt[i, :n] = torch.tensor([perm.pop() for _ in range(n)], dtype=torch.int32)
    return kc, vc, bt


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window,sink", [(0, None), (7, None), (0, 0.0), (7, 0.0), (300, 1.5),
                                         (16, -2.0)])
def test_windowed_attention_with_sink(dtype, window, sink):
    g = torch.Generator().manual_seed(3)
    heads, kv_heads, dim, vdim, bs = 4, 2, 24, 24, 4
    # (new rows, total length): a whole prompt, a portion, a two-token portion
    spec = [(9, 9), (5, 40), (2, 300), (17, 17)]
    ctxs = [s[1] for s in spec]
    kc, vc, bt = _paged(ctxs, bs, kv_heads, dim, vdim, dtype, g)
    qsl = torch.tensor([0] + list(torch.tensor([s[0] for s in spec]).cumsum(0)), dtype=torch.int32)
    lens = torch.tensor(ctxs, dtype=torch.int32)
    q = torch.randn(int(qsl[-1]), heads, dim, generator=g).to(dtype)
    want = ref.paged_attention(q, kc, vc, bt, qsl, lens, 0.3, window, sink)
    out = torch.empty(q.shape[0], heads, vdim, dtype=dtype, device=DEV)
    ops.gqa_attention_prefill(q.to(DEV), kc.to(DEV), vc.to(DEV), bt.to(DEV), qsl.to(DEV),
                              lens.to(DEV), 0.3, 17, out=out, window=window, sink=sink)
    _close(out, want, dtype, "portions")
    # one query per sequence, one padding row of length 0
    lens1 = torch.tensor(ctxs + [0], dtype=torch.int32)
    bt1 = torch.cat([bt, torch.zeros(1, bt.shape[1], dtype=torch.int32)])
    q1 = torch.randn(len(ctxs) + 1, heads, dim, generator=g).to(dtype)
    qsl1 = torch.arange(len(ctxs) + 2, dtype=torch.int32)
    want1 = ref.paged_attention(q1, kc, vc, bt1, qsl1, lens1, 0.3, window, sink)
    out1 = torch.empty(q1.shape[0], heads, vdim, dtype=dtype, device=DEV)
    ops.gqa_attention_decode(q1.to(DEV), kc.to(DEV), vc.to(DEV), bt1.to(DEV), lens1.to(DEV),
                             0.3, out=out1, window=window, sink=sink)
    _close(out1, want1, dtype, "single queries")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("d", [5, 16, 80])
def test_gates_and_squared_relu(dtype, d):
    g = torch.Generator().manual_seed(4)
    t, h = 7, 3
    o_hm = torch.randn(h, t, d, generator=g).to(dtype)          # head-major, as a bmm leaves it
    gate_h = torch.randn(t, h, generator=g).to(dtype)
    gate_e = torch.randn(t, h * d + 4, generator=g).to(dtype)[:, 4:].view(t, h, d)
    want = ref.sigmoid_gate_mul(o_hm.transpose(0, 1), gate_h)
    got = ops.sigmoid_gate_mul(o_hm.to(DEV).transpose(0, 1), gate_h.to(DEV))
    _close(got, want, dtype, "per head")
    o_tm = torch.randn(t, h, d, generator=g).to(dtype)
    want = ref.sigmoid_gate_mul(o_tm, gate_e)
    ged = torch.randn(t, h * d + 4).to(dtype).to(DEV)
    ged[:, 4:] = gate_e.reshape(t, h * d).to(DEV)
    got = ops.sigmoid_gate_mul(o_tm.to(DEV), ged[:, 4:].view(t, h, d))
    _close(got, want, dtype, "per element")

    x = torch.randn(t, h * d, generator=g).to(dtype) * 2
    bias = torch.randn(h * d, generator=g).to(dtype)
    cs = torch.rand(t, h, generator=g)
    for bb, sc in ((None, None), (bias, None), (None, cs), (bias, cs)):
        want = ref.relu2(x, bb, sc)
        got = ops.relu2(x.to(DEV), None if bb is None else bb.to(DEV),
                        None if sc is None else sc.to(DEV))
        _close(got, want, dtype, "relu2")


@pytest.mark.parametrize("n,real,top", [(12, 8, 4), (5, 5, 1), (3, 1, 3), (70, 64, 6),
                                        (300, 256, 8), (2, 0, 1)])
def test_router(n, real, top):
    g = torch.Generator().manual_seed(5)
    t = 33
    z = torch.randn(t, n, generator=g) * 2
    corr = torch.randn(n, generator=g) * 0.2
    want = ref.moe_route(z, corr, top, real)
    got = ops.moe_route(z.to(DEV), corr.to(DEV), top, real)
    assert torch.equal(got[2].cpu(), want[2]), "chosen experts"
    for a, b, what in zip(got[:2] + got[3:], want[:2] + want[3:], ("dense", "identity", "weights")):
        _close(a, b, torch.float32, what)
    # ties go to the lower index
    z0 = torch.zeros(2, n)
    got = ops.moe_route(z0.to(DEV), torch.zeros(n, device=DEV), top, real)
    assert got[2].cpu().tolist() == [list(range(top))] * 2


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [10, 64])
def test_expert_combine(dtype, width):
    g = torch.Generator().manual_seed(6)
    t, top, real = 6, 3, 4
    ids = torch.randint(0, real + 2, (t, top), generator=g, dtype=torch.int32)
    w = torch.rand(t, top, generator=g)
    pos = torch.randperm(t * top, generator=g).view(t, top).to(torch.int32)
    ye = torch.randn(t * top, width, generator=g).to(dtype)
    want = ref.moe_combine(ye, pos, ids, w, real)
    got = ops.moe_combine(ye.to(DEV), pos.to(DEV), ids.to(DEV), w.to(DEV), real)
    _close(got, want, dtype, "combine")


def test_grouped_expert_product():
    g = torch.Generator().manual_seed(7)
    e, k, n, t = 5, 128, 256, 300
    x = torch.randn(t, k, generator=g).to(torch.bfloat16)
    w = (torch.randn(e, n, k, generator=g) / k ** 0.5).to(torch.bfloat16)
    seg = torch.tensor([0, 40, 40, 200, 201, 280], dtype=torch.int32)   # 20 rows past the end
    for act in (None, "relu2"):
        want = ref.moe_gemm(x, w, seg, False, act)
        got = ops.moe_gemm(x.to(DEV), w.to(DEV), seg.to(DEV), gated=False, act=act)
        _close(got[:280], want[:280], torch.bfloat16, f"act {act}")


@pytest.mark.parametrize("dim", [64, 128])
@pytest.mark.parametrize("window,sink", [(0, 0.0), (1, 0.0), (33, None), (64, 0.0), (100, 1.0),
                                         (257, 0.0), (5000, -1.0)])
def test_windowed_attention_on_matrix_cores(dim, window, sink):
    """bf16 shapes that run the MFMA kernels: windows that end inside, at the
    edge of and beyond a key tile, portions that start mid-tile, a two-token
    portion, single queries with a padding row."""
    g = torch.Generator().manual_seed(8)
    dtype = torch.bfloat16
    heads, kv_heads, bs = 8, 2, 16
    spec = [(300, 300), (70, 391), (2, 130), (1 + 256, 700), (5, 5)]
    ctxs = [s[1] for s in spec]
    kc, vc, bt = _paged(ctxs, bs, kv_heads, dim, dim, dtype, g)
    news = torch.tensor([s[0] for s in spec])
    qsl = torch.tensor([0] + news.cumsum(0).tolist(), dtype=torch.int32)
    lens = torch.tensor(ctxs, dtype=torch.int32)
    q = torch.randn(int(qsl[-1]), heads, dim, generator=g).to(dtype)
    scale = dim ** -0.5
    want = ref.paged_attention(q, kc, vc, bt, qsl, lens, scale, window, sink)
    out = torch.empty(q.shape[0], heads, dim, dtype=dtype, device=DEV)
    ops.gqa_attention_prefill(q.to(DEV), kc.to(DEV), vc.to(DEV), bt.to(DEV), qsl.to(DEV),
                              lens.to(DEV), scale, int(news.max()), out=out, window=window,
                              sink=sink)
    _close(out, want, dtype, "portions")
    lens1 = torch.tensor(ctxs + [0], dtype=torch.int32)
    bt1 = torch.cat([bt, torch.zeros(1, bt.shape[1], dtype=torch.int32)])
    q1 = torch.randn(len(ctxs) + 1, heads, dim, generator=g).to(dtype)
    qsl1 = torch.arange(len(ctxs) + 2, dtype=torch.int32)
    want1 = ref.paged_attention(q1, kc, vc, bt1, qsl1, lens1, scale, window, sink)
    out1 = torch.empty(q1.shape[0], heads, dim, dtype=dtype, device=DEV)
    ops.gqa_attention_decode(q1.to(DEV), kc.to(DEV), vc.to(DEV), bt1.to(DEV), lens1.to(DEV),
                             scale, out=out1, window=window, sink=sink)
    _close(out1, want1, dtype, "single queries")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("t,top,real,extra,width", [(37, 3, 5, 2, 64), (300, 4, 16, 4, 40),
                                                    (1, 2, 2, 0, 7), (64, 1, 1, 3, 128)])
def test_pairs_grouped_by_expert(dtype, t, top, real, extra, width):
    g = torch.Generator().manual_seed(9)
    # distinct experts per token, as a router gives them
    ids = torch.stack([torch.randperm(real + extra, generator=g)[:top] for _ in range(t)]).to(torch.int32)
    h = torch.randn(t, width + 8, generator=g).to(dtype)[:, 8:]      # a column slice
    xs, pos, seg = ops.moe_sort(ids.to(DEV), real, h.to(DEV)[:, :] if width % 8 else h.to(DEV))
    _, _, seg_r = ref.moe_sort(ids, real, h)
    assert torch.equal(seg.cpu(), seg_r)
    xs, pos, seg = xs.cpu(), pos.cpu().long(), seg.cpu().tolist()
    taken = set()
    for i in range(t):
        for k in range(top):
            e = int(ids[i, k])
            if e >= real:
                continue
            p = int(pos[i, k])
            assert seg[e] <= p < seg[e + 1] and p not in taken     # its own row of its segment
            taken.add(p)
            assert torch.equal(xs[p], h[i])
    assert len(taken) == seg[-1]


@pytest.mark.parametrize("dim", [64, 128])
@pytest.mark.parametrize("n_new", [1, 2, 70])
@pytest.mark.parametrize("window", [33, 64, 100, 257, 0])
def test_window_edge_on_matrix_cores(dim, n_new, window):
    """bf16 MFMA kernels: one key that the last query points at, with a value of
    100, placed just inside and just outside the window, at the sequence's
    start and at tile borders; everything else is small noise."""
    import math

    ctx, bs, dtype = 300, 16, torch.bfloat16
    nb = (ctx + bs - 1) // bs
    table = list(range(nb - 1, -1, -1))
    places = {0, ctx - 1, 63, 64, 255, 256}
    if window:
        places |= {ctx - window, ctx - window - 1, ctx - window + 1}
    for at in sorted(places):
        g = torch.Generator().manual_seed(at)
        k = torch.randn(ctx, 1, dim, generator=g) * 0.02
        v = torch.randn(ctx, 1, dim, generator=g) * 0.02
        q = torch.randn(n_new, 2, dim, generator=g) * 0.02
        direction = torch.ones(dim) / math.sqrt(dim)
        k[at, 0] = 8.0 * direction
        v[at, 0] = 100.0
        q[-1, :] = 8.0 * direction
        k, v, q = k.to(dtype), v.to(dtype), q.to(dtype)
        kc = torch.zeros(nb, bs, 1, dim, dtype=dtype)
        vc = torch.zeros(nb, bs, 1, dim, dtype=dtype)
        for p in range(ctx):
            kc[table[p // bs], p % bs] = k[p]
            vc[table[p // bs], p % bs] = v[p]
        i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
        out = torch.empty(n_new, 2, dim, dtype=dtype, device=DEV)
        if n_new > 1:
            ops.gqa_attention_prefill(q.to(DEV), kc.to(DEV), vc.to(DEV), i32([table]),
                                      i32([0, n_new]), i32([ctx]), 1.0, n_new, out=out,
                                      window=window, sink=0.0)
        else:
            ops.gqa_attention_decode(q.to(DEV), kc.to(DEV), vc.to(DEV), i32([table]),
                                     i32([ctx]), 1.0, out=out, window=window, sink=0.0)
        lo = max(0, ctx - window) if window else 0
        s = k[lo:ctx, 0].double() @ q[-1, 0].double()
        e = torch.exp(s)
        want = (e / (1.0 + e.sum())) @ v[lo:ctx, 0].double()
        seen = at >= lo
        assert (float(want.abs().max()) > 50.0) == seen
        got = out[-1, 0].double().cpu()
        assert float((got - want).abs().max()) < 0.6, f"spike at {at}: {got[:3]} vs {want[:3]}"


@pytest.mark.parametrize("two_term", [False, True])
@pytest.mark.parametrize("rank,rot", [(64, 32), (256, 32)])
def test_latent_attention_two_term_weights(rank, rot, two_term):
    """The latent MFMA kernel with one or two bf16 terms per softmax weight
    against the reference, portions and single queries."""
    g = torch.Generator().manual_seed(10)
    dtype, heads, bs = torch.bfloat16, 4, 16
    spec = [(200, 200), (3, 150), (40, 333)]
    ctxs = [s[1] for s in spec]
    nb = sum((c + bs - 1) // bs for c in ctxs) + 2
    cache = (torch.randn(nb, bs, rank + rot, generator=g) * 0.5).to(dtype)
    perm = torch.randperm(nb, generator=g).tolist()
    width = max((c + bs - 1) // bs for c in ctxs)
    bt = torch.zeros(len(ctxs), width, dtype=torch.int32)
    for i, c in enumerate(ctxs):
        n = (c + bs - 1) // bs
        bt[i, :n] = torch.tensor([perm.pop() for _ in range(n)], dtype=torch.int32)
    news = [s[0] for s in spec]
    qsl = torch.tensor([0] + torch.tensor(news).cumsum(0).tolist(), dtype=torch.int32)
    lens = torch.tensor(ctxs, dtype=torch.int32)
    t = int(qsl[-1])
    ql = (torch.randn(t, heads, rank, generator=g) * 0.3).to(dtype)
    qr = (torch.randn(t, heads, rot, generator=g) * 0.3).to(dtype)
    want = ref.latent_attention(ql, qr, cache, bt, qsl, lens, 0.2, 0, None)
    out = torch.empty(t, heads, rank, dtype=dtype, device=DEV)
    ops.latent_attention_prefill(ql.to(DEV), qr.to(DEV), cache.to(DEV), bt.to(DEV), qsl.to(DEV),
                                 lens.to(DEV), 0.2, 0, None, max(news), out=out,
                                 two_term=two_term)
    _close(out, want, dtype, "portions")
    q1l, q1r = ql[:3].contiguous(), qr[:3].contiguous()
    want1 = ref.latent_attention(q1l, q1r, cache, bt, torch.arange(4, dtype=torch.int32), lens,
                                 0.2, 0, None)
    out1 = torch.empty(3, heads, rank, dtype=dtype, device=DEV)
    ops.latent_attention_decode(q1l.to(DEV), q1r.to(DEV), cache.to(DEV), bt.to(DEV),
                                lens.to(DEV), 0.2, 0, None, out=out1, two_term=two_term)
    _close(out1, want1, dtype, "single queries")
