"""HIP kernels of the token shift, query/key norm + half-split rotation +
cache write, chunk-masked attention with shared value heads, the differential
combination, grouped RMS norm, the HGRN2 recurrence, the sigmoid router and the
weighted gated activation against the plain-PyTorch reference ops, on sizes
that hit vector and scalar paths."""

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


def _i32(v):
    return torch.tensor(v, dtype=torch.int32)


# sequences of a step: rows per sequence, length after the step, slot
SEQS = [
    ([3, 1, 5], [3, 9, 12], [2, 0, 3]),          # new, single token, continued portion
    ([1, 1, 1, 1], [1, 20, 7, 2], [1, -1, 0, 3]),  # decode rows, one padding row
    ([40], [40], [1]),
    ([2, 0, 6], [10, 4, 6], [0, 2, 1]),          # a sequence that brings nothing
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [6, 96, 1000])
@pytest.mark.parametrize("case", range(len(SEQS)))
def test_token_shift(dtype, width, case):
    rows, lens, slots = SEQS[case]
    g = torch.Generator().manual_seed(case)
    t = sum(rows)
    loc = _i32([0] + torch.tensor(rows).cumsum(0).tolist())
    x = torch.randn(t, width, generator=g)
    w = torch.rand(width, generator=g)
    state = torch.randn(4, width, generator=g)
    sr = state.clone()
    want = ref.token_shift_state(x, w, sr, loc, _i32(lens), _i32(slots), dtype)
    sg = state.clone().to(DEV)
    got = ops.token_shift_state(x.to(DEV), w.to(DEV), sg, loc.to(DEV), _i32(lens).to(DEV),
                                _i32(slots).to(DEV), dtype)
    _close(got, want, dtype, "shifted rows")
    _close(sg, sr, torch.float32, "carried rows")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("pad", [3, 8])      # 8: rows stay 16-byte aligned (vector kernel)
@pytest.mark.parametrize("heads,kv_heads,v_heads,dim,vdim,rot", [
    (4, 2, 1, 8, 12, 4), (6, 6, 3, 64, 64, 64), (2, 2, 2, 70, 5, 0), (8, 2, 1, 128, 96, 32),
    (32, 8, 4, 128, 128, 128), (3, 1, 1, 32, 8, 0), (2, 2, 1, 256, 64, 256), (2, 1, 1, 512, 16, 512),
])
def test_qk_norm_rope_cache_write(dtype, heads, kv_heads, v_heads, dim, vdim, rot, pad):
    g = torch.Generator().manual_seed(3)
    t, bs, blocks = 9, 4, 6
    cols = heads * dim + kv_heads * dim + v_heads * vdim + pad
    proj = torch.randn(t, cols, generator=g).to(dtype)
    a, b = heads * dim, (heads + kv_heads) * dim
    c = b + v_heads * vdim
    qw = torch.rand(dim, generator=g) + 0.5
    kw = torch.rand(dim, generator=g) + 0.5
    pos = torch.randint(0, 3000, (t,), generator=g)
    inv = torch.rand(max(rot, 2) // 2, generator=g)
    slots = torch.randperm(bs * blocks, generator=g)[:t]
    slots[2] = -1

    def run(dev, fn):
        p = proj.to(dev)
        kc = torch.zeros(blocks, bs, kv_heads, dim, dtype=dtype, device=dev)
        vc = torch.zeros(blocks, bs, v_heads, vdim, dtype=dtype, device=dev)
        q = fn(p[:, :a].view(t, heads, dim), p[:, a:b].view(t, kv_heads, dim),
               p[:, b:c].view(t, v_heads, vdim), qw.to(dev), kw.to(dev), 1e-6,
               pos.to(dev), inv.to(dev), rot, kc, vc, slots.to(dev))
        return q, kc, vc

    want = run("cpu", ref.qk_norm_rope_cache_write)
    got = run(DEV, ops.qk_norm_rope_cache_write)
    for gg, ww, what in zip(got, want, ("queries", "key cache", "value cache")):
        _close(gg, ww, dtype, what)


def _paged(ctx_lens, kv_heads, v_heads, dim, vdim, bs, dtype, g):
    nblk = [(n + bs - 1) // bs for n in ctx_lens]
    total = sum(nblk) + 2
    order = torch.randperm(total, generator=g).tolist()
    tables = torch.zeros(len(ctx_lens), max(nblk), dtype=torch.int32)
    for i, n in enumerate(nblk):
        for j in range(n):
            tables[i, j] = order.pop()
    kc = torch.randn(total, bs, kv_heads, dim, generator=g).to(dtype)
    vc = torch.randn(total, bs, v_heads, vdim, generator=g).to(dtype)
    return kc, vc, tables


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("chunk", [0, 5, 16, 300])
@pytest.mark.parametrize("heads,kv_heads,v_heads,dim,vdim", [
    (8, 2, 1, 16, 24), (4, 4, 2, 64, 64), (6, 2, 2, 40, 300),
    (8, 4, 2, 128, 128), (16, 2, 1, 128, 128), (4, 2, 1, 64, 64),   # matrix-core shapes
])
def test_chunk_attention(dtype, chunk, heads, kv_heads, v_heads, dim, vdim):
    g = torch.Generator().manual_seed(11)
    bs = 4
    new = [7, 1, 33, 2]
    ctx = [7, 40, 35, 290]
    kc, vc, tables = _paged(ctx, kv_heads, v_heads, dim, vdim, bs, dtype, g)
    qsl = _i32([0] + torch.tensor(new).cumsum(0).tolist())
    q = torch.randn(sum(new), heads, dim, generator=g).to(dtype)
    want = ref.chunk_attention(q, kc, vc, tables, qsl, _i32(ctx), 0.3, chunk)
    out = torch.empty(sum(new), heads, vdim, dtype=torch.float32, device=DEV)
    ops.chunk_attention_prefill(q.to(DEV), kc.to(DEV), vc.to(DEV), tables.to(DEV),
                                qsl.to(DEV), _i32(ctx).to(DEV), 0.3, max(new), chunk, out)
    _close(out, want, dtype, "portions")
    # one query per sequence, the second a padding row
    ctx1 = [17, 0, 35, 290]
    q1 = torch.randn(4, heads, dim, generator=g).to(dtype)
    want = ref.chunk_attention(q1, kc, vc, tables, _i32([0, 1, 2, 3, 4]), _i32(ctx1), 0.3,
                               chunk)
    out = torch.empty(4, heads, vdim, dtype=torch.float32, device=DEV)
    ops.chunk_attention_decode(q1.to(DEV), kc.to(DEV), vc.to(DEV), tables.to(DEV),
                               _i32(ctx1).to(DEV), 0.3, chunk, out)
    _close(out, want, dtype, "single queries")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("chunk", [0, 64, 100, 257, 1000])
@pytest.mark.parametrize("new,ctx", [([300, 40], [330, 700]), ([513], [513]), ([2, 260], [130, 261])])
def test_chunk_attention_long_portions(dtype, chunk, new, ctx):
    """Portions that span several query and key tiles of the matrix-core
    kernel, chunk edges inside tiles and on their borders."""
    heads, kv_heads, v_heads, dim = 4, 2, 1, 128
    g = torch.Generator().manual_seed(12)
    kc, vc, tables = _paged(ctx, kv_heads, v_heads, dim, dim, 16, dtype, g)
    qsl = _i32([0] + torch.tensor(new).cumsum(0).tolist())
    q = torch.randn(sum(new), heads, dim, generator=g).to(dtype)
    want = ref.chunk_attention(q, kc, vc, tables, qsl, _i32(ctx), 0.1, chunk)
    out = torch.empty(sum(new), heads, dim, dtype=torch.float32, device=DEV)
    ops.chunk_attention_prefill(q.to(DEV), kc.to(DEV), vc.to(DEV), tables.to(DEV),
                                qsl.to(DEV), _i32(ctx).to(DEV), 0.1, max(new), chunk, out)
    _close(out, want, dtype, "portions")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,vdim,gate", [(3, 10, True), (4, 64, True), (2, 200, False), (2, 300, True)])
def test_diff_combine(dtype, heads, vdim, gate):
    g = torch.Generator().manual_seed(5)
    t = 11
    a = torch.randn(t, 2, heads, vdim, generator=g)
    proj = torch.randn(t, heads + 5, generator=g).to(dtype)
    gt = proj[:, 5:] if gate else None
    want = ref.diff_combine(a, 0.37, 0.8, 1e-6, gt, dtype)
    pg = proj.to(DEV)
    got = ops.diff_combine(a.to(DEV), 0.37, 0.8, 1e-6, pg[:, 5:] if gate else None, dtype)
    _close(got, want, dtype, "combined heads")


@pytest.mark.parametrize("in_dtype,out_dtype", [
    (torch.float32, torch.float32), (torch.float32, torch.bfloat16),
    (torch.bfloat16, torch.bfloat16)])
@pytest.mark.parametrize("groups,gsize", [(1, 80), (4, 64), (3, 7), (2, 300), (1, 1536), (2, 256)])
def test_group_rms_norm(in_dtype, out_dtype, groups, gsize):
    g = torch.Generator().manual_seed(6)
    y = (torch.randn(7, groups * gsize, generator=g) * 3).to(in_dtype)
    w = torch.rand(groups * gsize, generator=g) + 0.5
    want = ref.group_rms_norm(y, w, groups, 1e-6, out_dtype)
    got = ops.group_rms_norm(y.to(DEV), w.to(DEV), groups, 1e-6, out_dtype)
    _close(got, want, out_dtype, "normed groups")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,dim,vdim", [(2, 8, 12), (4, 32, 64), (3, 20, 7), (2, 128, 256),
                                            (1, 264, 40)])
@pytest.mark.parametrize("case", range(len(SEQS)))
def test_hgrn2_scan(dtype, heads, dim, vdim, case):
    rows, lens, slots = SEQS[case]
    g = torch.Generator().manual_seed(case + 20)
    t = sum(rows)
    loc = _i32([0] + torch.tensor(rows).cumsum(0).tolist())
    a = heads * dim
    proj = torch.randn(t, 2 * a + heads * vdim, generator=g).to(dtype)
    fb = torch.randn(a, generator=g)
    lower = torch.rand(a, generator=g)
    state = torch.randn(4, heads, vdim, dim, generator=g)

    def run(dev, fn):
        p, st = proj.to(dev), state.clone().to(dev)
        o = fn(p[:, :a].view(t, heads, dim), p[:, a:2 * a].view(t, heads, dim),
               p[:, 2 * a:].view(t, heads, vdim), fb.to(dev), lower.to(dev), st,
               loc.to(dev), _i32(lens).to(dev), _i32(slots).to(dev))
        return o, st

    ow, sw = run("cpu", ref.hgrn2_scan)
    og, sg = run(DEV, ops.hgrn2_scan)
    _close(og, ow, torch.float32, "outputs")
    _close(sg, sw, torch.float32, "state")


@pytest.mark.parametrize("experts,top", [(5, 1), (12, 3), (64, 8), (130, 2), (4, 4)])
def test_sigmoid_router(experts, top):
    g = torch.Generator().manual_seed(8)
    z = torch.randn(37, experts, generator=g) * 2
    dw, iw, ww = ref.moe_route_sigmoid(z, top)
    dg, ig, wg = ops.moe_route_sigmoid(z.to(DEV), top)
    assert torch.equal(ig.cpu().sort(dim=-1).values, iw.sort(dim=-1).values)
    _close(dg, dw, torch.float32, "dense weights")
    _close(wg.sum(-1), ww.sum(-1), torch.float32, "weights")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("experts,ff", [(3, 10), (12, 64), (2, 129)])
def test_silu_mul_scaled(dtype, experts, ff):
    g = torch.Generator().manual_seed(9)
    t = 6
    gu = torch.randn(t, experts * 2 * ff, generator=g).to(dtype)
    sc = torch.rand(t, experts, generator=g)
    sc[sc < 0.4] = 0.0
    want = ref.silu_mul_scaled(gu, sc)
    got = ops.silu_mul_scaled(gu.to(DEV), sc.to(DEV))
    _close(got, want, dtype, "activations")


@pytest.mark.parametrize("dtype", DTYPES)
def test_stream_add_norm_with_layer_scale_and_cast(dtype):
    g = torch.Generator().manual_seed(10)
    for width in (6, 192, 1000):
        x = torch.randn(5, width, generator=g)
        y = torch.randn(5, width, generator=g).to(dtype)
        w = torch.rand(width, generator=g) + 0.5
        ls = torch.randn(width, generator=g)
        xr = x.clone()
        ref.stream_add_rms_norm(xr, y, w, 1e-6, 1.0, ls)
        xg = x.clone().to(DEV)
        h = ops.stream_add_rms_norm(xg, y.to(DEV), w.to(DEV), 1e-6, 1.0,
                                    layer_scale=ls.to(DEV), cast_dtype=dtype)
        _close(xg, xr, torch.float32, "stream")
        _close(h, xr.to(dtype), dtype, "rounded stream")
